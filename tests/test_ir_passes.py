"""C++ unit tests against the library's own headers, compiled and run here (no GPU needed): the GPU IR passes
(csrc/optim) on hand-built loop nests (tests/cpp/test_ir_passes.cc), the host-stub pool beyond its pre-compiled
trampolines (tests/cpp/test_host_stubs.cc) and the placement of a program's tensors in one allocation
(tests/cpp/test_memory_plan.cc)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _build_and_run(tmp_path, name):
    lib_dir = os.path.join(ROOT, "cinn_amd", "lib")
    assert os.path.exists(os.path.join(lib_dir, "libcinn_hip.so")), "build the library first (__graft_entry__.build())"
    exe = str(tmp_path / name)
    cmd = ["g++", "-std=c++17", "-O1", "-I" + os.path.join(ROOT, "cinn_amd", "csrc"), "-I" + os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "cpp", name + ".cc"), "-L" + lib_dir, "-lcinn_hip",
           "-Wl,-rpath," + lib_dir, "-Wl,-rpath,/opt/rocm/lib", "-o", exe]
    built = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert built.returncode == 0, built.stderr
    ran = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert ran.returncode == 0 and ran.stdout.strip().endswith("ok"), ran.stdout + ran.stderr


def test_gpu_ir_passes_on_hand_built_loop_nests(tmp_path):
    _build_and_run(tmp_path, "test_ir_passes")


def test_host_stubs_beyond_the_precompiled_trampolines(tmp_path):
    """4096 + 700 live stubs: the first 4096 are pre-compiled trampolines, the rest generated thunks; each calls its own
    closure, released thunks are reused (the reference JIT-compiles host stubs with LLVM and has no such bound,
    cinn/backends/llvm/execution_engine.cc)."""
    _build_and_run(tmp_path, "test_host_stubs")


def test_memory_plan_never_overlaps_values_that_are_alive_together(tmp_path):
    _build_and_run(tmp_path, "test_memory_plan")
