"""The GPU IR passes (csrc/optim) on hand-built loop nests: a C++ program against the library's own IR headers,
compiled and run here (no GPU needed).  The cases are in tests/cpp/test_ir_passes.cc."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_gpu_ir_passes_on_hand_built_loop_nests(tmp_path):
    lib_dir = os.path.join(ROOT, "cinn_amd", "lib")
    assert os.path.exists(os.path.join(lib_dir, "libcinn_hip.so")), "build the library first (__graft_entry__.build())"
    exe = str(tmp_path / "test_ir_passes")
    cmd = ["g++", "-std=c++17", "-O1", "-I" + os.path.join(ROOT, "cinn_amd", "csrc"), "-I" + os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "cpp", "test_ir_passes.cc"), "-L" + lib_dir, "-lcinn_hip",
           "-Wl,-rpath," + lib_dir, "-Wl,-rpath,/opt/rocm/lib", "-o", exe]
    built = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert built.returncode == 0, built.stderr
    ran = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert ran.returncode == 0 and ran.stdout.strip().endswith("ok"), ran.stdout + ran.stderr
