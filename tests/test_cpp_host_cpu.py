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


def test_cpp_header_compiles_standalone_with_warnings_as_errors(tmp_path):
    src = tmp_path / "t.cpp"
    src.write_text('#include "fandhe_rocm.hpp"\nint main() { return 0; }\n')
    subprocess.check_call(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-fsyntax-only",
                           "-I", os.path.join(ROOT, "include"), str(src)])
