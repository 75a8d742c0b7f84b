"""The C-ABI library loads, exports every symbol the public headers declare, and lays out the ABI structs
exactly like the reference's cinn_runtime.h (checked against the probe compiled from the reference's own
sources when it is present, and against the documented numbers otherwise).  No compute calls here."""
import ctypes
import os
import re

import numpy as np
import pytest

import oracle
from cinn_amd import _lib, runtime

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(cinn_[a-z0-9_]+)\s*\(", text)
    return sorted(set(n for n in names if not n.endswith("_t")))


@pytest.mark.parametrize("header", ["cinn_hip_runtime.h", "cinn_amd_api.h"])
def test_library_exports_every_declared_symbol(header):
    lib = _lib.load()
    names = _declared_functions(header)
    assert len(names) > 10
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, "declared in include/%s but not exported: %s" % (header, missing)


def test_reference_intrinsic_names_present():
    # the names JIT'd host code of the reference resolves by string (cuda_intrinsics.cc:404-733)
    lib = _lib.load()
    for name in ["cinn_call_cuda_kernel", "cinn_call_cublas", "cinn_call_batched_cublas",
                 "cinn_call_cudnn_conv2d_forward", "cinn_call_cudnn_pool2d_forward",
                 "cinn_call_cudnn_softmax_forward", "cinn_call_cuda_memset", "cinn_call_cuda_memcpy"]:
        assert hasattr(lib, name), name


def test_every_declared_intrinsic_can_be_called_from_a_host_stub():
    # every cinn_call_* of the header has a registered prototype, so a compiled program's host function can call it
    # (REGISTER_EXTERN_FUNC_HELPER list, cinn/runtime/cuda/cuda_intrinsics.cc:404-733)
    lib = _lib.load()
    registered = set(_lib.read_string(lib.cinn_amd_extern_api_names).split(","))
    # (the status-returning entry point for callers that cannot allocate is not a host-stub prototype)
    declared = [n for n in _declared_functions("cinn_hip_runtime.h")
                if n.startswith("cinn_call_") and not n.endswith("_noalloc")]
    assert len(declared) >= 14
    assert not [n for n in declared if n not in registered], registered
    # a stub is a real function pointer; wrong arity and unknown names are reported, not executed
    fn = ctypes.c_void_p()
    _lib.check(lib.cinn_amd_host_stub_create(b"cinn_call_cuda_memcpy", b"i:16", ctypes.byref(fn)))
    assert fn.value
    _lib.check(lib.cinn_amd_host_stub_release(fn))
    assert lib.cinn_amd_host_stub_create(b"cinn_call_cuda_memcpy", b"i:16,i:3", ctypes.byref(fn)) != 0
    assert "wrong number of arguments" in lib.cinn_amd_last_error().decode()
    assert lib.cinn_amd_host_stub_create(b"cinn_call_nothing", b"", ctypes.byref(fn)) != 0
    assert lib.cinn_amd_host_stub_create(b"cinn_call_cuda_memcpy", b"x:1", ctypes.byref(fn)) != 0


def test_struct_layout_documented_numbers():
    assert ctypes.sizeof(runtime.cinn_type_t) == 12
    assert ctypes.sizeof(runtime.cinn_buffer_t) == 120
    assert runtime.cinn_buffer_t.memory.offset == 16
    assert runtime.cinn_buffer_t.type.offset == 32
    assert runtime.cinn_buffer_t.dimensions.offset == 44
    assert runtime.cinn_buffer_t.dims.offset == 48
    assert runtime.cinn_buffer_t.memory_size.offset == 88
    assert ctypes.sizeof(runtime.cinn_pod_value_t) == 16
    assert runtime.cinn_pod_value_t.value_.offset == 8


needs_ref = pytest.mark.skipif(oracle.ref is None, reason="oracle/_ref was not built (reference tree absent)")


@needs_ref
def test_struct_layout_against_reference_build():
    out = (ctypes.c_long * 10)()
    oracle.ref.ref_abi_layout(out)
    b = runtime.cinn_buffer_t
    assert list(out) == [ctypes.sizeof(runtime.cinn_type_t), ctypes.sizeof(b), b.memory.offset, b.type.offset,
                         b.dimensions.offset, b.dims.offset, b.memory_size.offset,
                         ctypes.sizeof(runtime.cinn_pod_value_t), b.flag.offset, b.align.offset]


@needs_ref
def test_pod_type_codes_against_reference_build():
    codes = (ctypes.c_int * 17)()
    oracle.ref.ref_pod_type_codes(codes)
    # CINN_POD_* of include/cinn_hip_runtime.h, same order
    assert list(codes) == list(range(17))
    t = (ctypes.c_long * 3)()
    expect = {0: (2, 32), 1: (2, 16), 2: (4, 16), 3: (0, 32), 4: (0, 1), 5: (2, 64), 6: (0, 64)}
    names = {0: "float32", 1: "float16", 2: "bfloat16", 3: "int32", 4: "bool", 5: "float64", 6: "int64"}
    for which, (code, bits) in expect.items():
        assert oracle.ref.ref_type_of(which, t) == 0
        # lanes is 0: the reference's constructors pass num_asterisks in the lanes slot
        assert (t[0], t[1], t[2]) == (code, bits, 0)
        assert runtime._TYPE_CODES[names[which]] == (code, bits)


@needs_ref
def test_buffers_and_pods_filled_by_the_library_read_back_through_reference_accessors():
    lib = _lib.load()
    buf = runtime.cinn_buffer_t()
    dims = (ctypes.c_int32 * 3)(4, 5, 6)
    fake_ptr = ctypes.c_void_p(0x7F0012345600)
    lib.cinn_hip_buffer_init(ctypes.byref(buf), fake_ptr, 2, 16, dims, 3)
    out = (ctypes.c_long * 15)()
    oracle.ref.ref_read_buffer(ctypes.byref(buf), out)
    assert list(out)[:10] == [2, 16, 0, 3, 120, 240, 1, 4, 5, 6]
    pods = (runtime.cinn_pod_value_t * 2)()
    lib.cinn_hip_pod_from_buffer(ctypes.byref(pods[0]), ctypes.byref(buf))
    lib.cinn_hip_pod_from_int32(ctypes.byref(pods[1]), 77)
    oracle.ref.ref_read_pod_buffer_memory.restype = ctypes.c_void_p
    assert oracle.ref.ref_read_pod_buffer_memory(pods, 0) == fake_ptr.value
    assert oracle.ref.ref_read_pod_type_code(pods, 0) == 7
    assert oracle.ref.ref_read_pod_type_code(pods, 1) == 0


def test_target_info_defaults_describe_gfx950():
    from cinn_amd.common import target_info
    info = target_info()
    assert info["wavefront_size"] == 64
    assert info["max_threads_per_block"] == 1024
    assert info["arch"].startswith("gfx9")
    if not info["from_device"]:
        assert info["multi_processor_count"] == 256 and info["lds_bytes_per_multi_processor"] == 160 * 1024


def test_device_library_text_is_embedded():
    text = _lib.load().cinn_hip_device_lib_source().decode()
    for needle in ["CINN_BLOCK_REDUCE_INTERNAL_IMPL", "CINN_HIP_WAVE_ALLREDUCE", "cinn_hip_copy_vec",
                   "cinn_hip_argmax_combine", "__ocml_exp_f32", "__builtin_amdgcn_update_dpp"]:
        assert needle in text


def test_rtc_reports_compile_errors_with_a_log():
    with pytest.raises(_lib.CinnError) as e:
        runtime.rtc_compile('extern "C" __global__ void k(float* a) { a[0] = undeclared_symbol; }')
    assert "undeclared_symbol" in str(e.value)


def test_rtc_compiles_for_gfx950_without_a_gpu():
    src = ('#include "cinn_hip_runtime_source.h"\n'
           'extern "C" __global__ void k(float* a) { a[threadIdx.x] = '
           'cinn_wave_shuffle_sum_fp32_internal(a[threadIdx.x]); }')
    image = runtime.rtc_compile(src)
    assert image[:4] == b"\x7fELF" and len(image) > 1000
    # same source again is served from the cache and is byte-identical
    assert runtime.rtc_compile(src) == image


def test_code_objects_are_kept_on_disk_between_processes(tmp_path):
    """FLAGS_cinn_hip_code_cache_dir: the first process compiles and stores <hash>.hsaco; a later process is served
    from that file (shown by editing the file's payload: the edited bytes come back); a file whose header does not fit
    is ignored and replaced."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cache = tmp_path / "code_cache"
    script = ("import sys; from cinn_amd import runtime; "
              "src = 'extern \"C\" __global__ void k(float* a) { a[threadIdx.x] += 1.0f; }'; "
              "sys.stdout.buffer.write(runtime.rtc_compile(src, with_device_lib=False))")
    env = dict(os.environ, FLAGS_cinn_hip_code_cache_dir=str(cache), PYTHONPATH=root)

    def compile_in_new_process():
        out = subprocess.run([sys.executable, "-c", script], cwd=root, env=env, capture_output=True, timeout=300)
        assert out.returncode == 0, out.stderr.decode()
        return out.stdout

    image = compile_in_new_process()
    assert image[:4] == b"\x7fELF"
    files = list(cache.glob("*.hsaco"))
    assert len(files) == 1 and not list(cache.glob("*.tmp.*"))
    blob = files[0].read_bytes()
    assert blob[32:] == image and int.from_bytes(blob[24:32], "little") == len(image)
    # a payload edited in place comes back from the next process: the file, not hiprtc, served it
    edited = bytearray(blob)
    edited[-1] ^= 0xFF
    files[0].write_bytes(bytes(edited))
    assert compile_in_new_process() == bytes(edited[32:])
    # truncated file: size in the header no longer fits -> recompiled and rewritten
    files[0].write_bytes(blob[:-7])
    assert compile_in_new_process() == image
    assert files[0].read_bytes() == blob
    # a different source gets a file of its own
    script2 = script.replace("+= 1.0f", "+= 2.0f")
    out = subprocess.run([sys.executable, "-c", script2], cwd=root, env=env, capture_output=True, timeout=300)
    assert out.returncode == 0 and len(list(cache.glob("*.hsaco"))) == 2


def test_bench_refuses_more_than_one_gpu():
    """the measured path has no cross-GPU work: bench.py --gpus N > 1 exits with a message instead of a number"""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in (r.stdout + r.stderr)
    assert not any(line.startswith("{") for line in r.stdout.splitlines())


FLOAT_FNS = ["sin", "cos", "tan", "sinh", "cosh", "tanh", "asin", "acos", "atan", "asinh", "acosh", "atanh", "ceil", "round",
             "trunc", "abs", "floor", "log", "log2", "log10", "exp", "erf", "sigmoid", "sqrt", "rsqrt", "cbrt"]


def reference_spelling_calls():
    """One call of every device-library name an unchanged CINN lowering can emit (the cinn_nvgpu_<fn>_<type> table of
    cinn/runtime/cuda/cinn_cuda_runtime_source.cuh:12-370 and the cinn_cuda_* / counting / index helpers of :619-843),
    as statements that accumulate into `double acc`."""
    calls = []
    ctype = {"fp32": "float", "fp64": "double", "fp16": "float16", "bf16": "bfloat16"}
    for sfx, t in ctype.items():
        v = "(%s)0.5f" % t
        for fn in FLOAT_FNS:
            calls.append("acc += (double)(float)cinn_nvgpu_%s_%s(%s);" % (fn, sfx, v))
        for fn in ("isfinite", "isinf", "isnan"):
            calls.append("acc += cinn_nvgpu_%s_%s(%s) ? 1.0 : 0.0;" % (fn, sfx, v))
        for fn in ("pow", "mod"):
            calls.append("acc += (double)(float)cinn_nvgpu_%s_%s(%s, (%s)3.0f);" % (fn, sfx, v, t))
    ints = {"uint8": "uint8_t", "int8": "int8_t", "int16": "int16_t", "int32": "int", "int64": "long long"}
    for sfx, t in ints.items():
        for fn in ("bitwise_and", "bitwise_or", "bitwise_xor", "logical_right_shift"):
            calls.append("acc += (double)cinn_nvgpu_%s_%s((%s)12, (%s)2);" % (fn, sfx, t, t))
        calls.append("acc += (double)cinn_nvgpu_bitwise_not_%s((%s)12);" % (sfx, t))
    for fn in ("bitwise_and", "bitwise_or", "bitwise_xor"):
        calls.append("acc += cinn_nvgpu_%s_bool(true, false) ? 1.0 : 0.0;" % fn)
    calls.append("acc += cinn_nvgpu_bitwise_not_bool(true) ? 1.0 : 0.0;")
    for fn in ("pow", "left_shift", "right_shift", "max", "min", "mod"):
        calls.append("acc += (double)cinn_nvgpu_%s_int32(7, 2);" % fn)
    for fn in ("clz", "popc", "trunc"):
        calls.append("acc += (double)cinn_nvgpu_%s_int32(7);" % fn)
        calls.append("acc += (double)cinn_nvgpu_%s_int64(7ll);" % fn)
    calls.append("acc += (double)cinn_nvgpu_mod_int64(7ll, 2ll) + (double)cinn_nvgpu_pow_int64(7ll, 2ll);")
    calls.append("acc += cinn_cuda_find_int(ibuf, 4, 1) + cinn_cuda_find_float(fbuf, 4, 1.0f);")
    calls.append("acc += cinn_cuda_find_int_nd(ibuf, 2, 1, 0, 2) + cinn_cuda_find_float_nd(fbuf, 2, 1.0f, 0, 2);")
    calls.append("acc += cinn_cuda_find_int_from(ibuf, 4, 1, 1) + cinn_cuda_find_float_from(fbuf, 4, 1.0f, 1);")
    calls.append("acc += cinn_nvgpu_next_smallest_int32(ibuf, 4, 0, 0, 1);")
    for sfx, buf, v in (("fp32", "fbuf", "1.0f"), ("fp64", "dbuf", "1.0"), ("int32", "ibuf", "1"), ("int64", "lbuf", "1ll"),
                        ("fp16", "hbuf", "(float16)1.0f")):
        calls.append("acc += cinn_nvgpu_lt_num_%s(%s, 4, %s, 0, 1) + cinn_nvgpu_gt_num_%s(%s, 4, %s, 0, 1);" % (sfx, buf, v, sfx, buf, v))
    for sfx, buf, v in (("fp32", "fbuf", "1.0f"), ("fp64", "dbuf", "1.0"), ("int32", "ibuf", "1"), ("int64", "lbuf", "1ll"),
                        ("fp16", "hbuf", "(float16)1.0f"), ("int8", "cbuf", "(int8_t)1"), ("bool", "bbuf", "true")):
        calls.append("acc += (double)(float)cinn_nvgpu_index_add_%s(%s, 1, %s, 0, 1, ibuf, 4);" % (sfx, v, buf))
    calls.append("acc += cinn_cuda_resize_bilinear(ibuf, 1, 2, 2, 4, 4, 0, 0, 1, 1) + cinn_cuda_resize_bicubic(ibuf, 1, 2, 2, 4, 4, 0, 0, 1, 1);")
    return calls


def test_device_library_defines_the_reference_spellings():
    calls = reference_spelling_calls()
    assert len(calls) > 180
    src = ('#include "cinn_hip_runtime_source.h"\n'
           'extern "C" __global__ void every_name(int* ibuf, float* fbuf, double* dbuf, long long* lbuf, float16* hbuf, '
           'int8_t* cbuf, bool* bbuf, double* out) {\n  double acc = 0.0;\n  ' + "\n  ".join(calls) +
           "\n  out[threadIdx.x] = acc;\n}\n")
    image = runtime.rtc_compile(src)
    assert image[:4] == b"\x7fELF"


def test_chunked_patch_kernel_wait_counts_match_a_simulation_of_its_issue_order():
    """conv3x3_patch_chunks_kernel's feeding wavefronts wait with `s_waitcnt vmcnt(n)` before every barrier: loads
    complete in issue order, so "at most n in flight" means that everything issued earlier than the last n loads has
    landed.  What must have landed at the barrier that closes K step s: filter stage s + 2 (its fragments are read
    during step s + 1) and, at tap 7, the next chunk's patch (read in the last rows of tap 8).  n comes from a closed
    formula in the kernel; here the issue order is replayed load by load (the first patch, the nine stages of chunk 0,
    then per K step the next chunk's patch loads and the stage nine steps ahead) and the exact largest safe n is
    counted at every barrier.  The formula may never exceed it (a race), and equals it."""
    lib = _lib.load()
    lib.cinn_hip_conv_patch_loads_in_flight.argtypes = [ctypes.c_int] * 4
    lib.cinn_hip_conv_patch_loads_in_flight.restype = ctypes.c_int
    taps, ring, patch_steps, stage_loads, ahead = 9, 9, 4, 2, 2
    for chunks in range(2, 7):
        total = chunks * taps
        for per_step in (2, 3):
            log = [("patch", 0)] * (per_step * patch_steps)
            for st in range(ring):
                log += [("stage", st)] * stage_loads
            for c in range(chunks):
                last = c == chunks - 1
                for t in range(taps):
                    if last and t == taps - 1:
                        break  # the last K step has no barrier
                    s = c * taps + t
                    needed = [("stage", min(s + ahead, total - 1))]
                    if not last and t == taps - ahead:
                        needed.append(("patch", c + 1))
                    newest = max(max(i for i, e in enumerate(log) if e == what) for what in needed)
                    exact = len(log) - 1 - newest
                    got = lib.cinn_hip_conv_patch_loads_in_flight(t, int(c == 0), int(last), per_step)
                    assert got == exact, (chunks, per_step, c, t, got, exact)
                    assert got <= 40  # the kernel's table of s_waitcnt immediates
                    if not last:
                        if t < patch_steps:
                            log += [("patch", c + 1)] * per_step
                        log += [("stage", s + ring)] * stage_loads
