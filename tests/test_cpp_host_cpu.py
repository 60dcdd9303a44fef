"""The C++ host layer (include/fandhe_rocm.hpp) without a device: its own test program covers page allocation
order, configuration checks, generate and the scheduler over a toy decoder (tests/cpp/host_cpu_test.cpp)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "fandhe_ai_amd", "lib")


def host_binary(name):
    path = os.path.join(LIB, name)
    if not os.path.exists(path):                    # built by __graft_entry__.build(); only if nothing is there
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "fandhe_ai_amd", "csrc"), os.path.join("..", "lib", name)])
    return path


def test_cpp_host_layer_on_a_toy_decoder():
    r = subprocess.run([host_binary("host_cpu_test")], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "checks ok" in r.stdout


def test_kernel_index_arithmetic_on_the_host():
    """The functions the large-tile GEMM, the streamed attention and the split-k linears use for their block, tile,
    stage, LDS and workspace offsets (fandhe_ai_amd/csrc/index_models.hpp), walked on the host for every instantiation:
    offsets in bounds, a stage's bytes where the operand reads expect them, every output written exactly once
    (tests/cpp/host_index_model_test.cpp)."""
    r = subprocess.run([host_binary("host_index_model_test")], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "checks ok" in r.stdout


def test_cpp_header_compiles_standalone_with_warnings_as_errors(tmp_path):
    src = tmp_path / "t.cpp"
    src.write_text('#include "fandhe_rocm.hpp"\nint main() { return 0; }\n')
    subprocess.check_call(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-fsyntax-only",
                           "-I", os.path.join(ROOT, "include"), str(src)])


def test_cpp_safetensors_reader_format_and_error_cases():
    r = subprocess.run([host_binary("host_safetensors_test")], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "checks ok" in r.stdout


def test_cpp_safetensors_reader_reads_what_the_python_writer_wrote(tmp_path):
    """A mixed-dtype file from the Python writer (bit-identical to the safetensors library's): the C++ reader must
    report the same dtypes and shapes and promote to the same float32 values as the Python reader."""
    import json
    import sys

    import numpy as np
    sys.path.insert(0, ROOT)
    try:
        from fandhe_ai_amd import safetensors_io as sio
    except ImportError as e:                               # the ctypes binding needs the library next to it
        import pytest
        pytest.skip(str(e))
    rng = np.random.default_rng(4)
    tensors = {
        "w.f32": sio.TypedTensor("F32", (3, 5), rng.standard_normal((3, 5)).astype(np.float32)),
        "w.f16": sio.TypedTensor("F16", (7,), (rng.standard_normal(7) * 100).astype(np.float16)),
        "w.bf16": sio.TypedTensor("BF16", (2, 2, 2), (rng.standard_normal(8).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16).reshape(2, 2, 2)),
        "w.f64": sio.TypedTensor("F64", (4,), rng.standard_normal(4)),
        "w.i32": sio.TypedTensor("I32", (3,), np.array([-5, 0, 2 ** 31 - 1], np.int32)),
        "w.i64": sio.TypedTensor("I64", (2,), np.array([-2 ** 40, 2 ** 53 + 1], np.int64)),
        "w.bool": sio.TypedTensor("BOOL", (5,), np.array([1, 0, 0, 1, 1], np.bool_)),
        "w.empty": sio.TypedTensor("F32", (0, 9), np.zeros((0, 9), np.float32)),
        "w.scalar": sio.TypedTensor("F32", (), np.array(2.5, np.float32)),
    }
    path = tmp_path / "mixed.safetensors"
    sio.save_safetensors_typed(str(path), tensors)
    r = subprocess.run([host_binary("host_safetensors_test"), str(path)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    got = json.loads(r.stdout)
    want = sio.load_safetensors_typed(str(path))
    assert sorted(got) == sorted(want)
    for name, t in want.items():
        g = got[name]
        assert g["dtype"] == t.dtype and tuple(g["shape"]) == tuple(t.shape), name
        v = t.to_f32().ravel()
        total = 0.0
        for x in v:                                         # same values, summed in double in file order
            total += float(x)
        assert g["sum"] == total, name
        if v.size:
            assert np.float32(g["first"]) == v[0] and np.float32(g["last"]) == v[-1], name
