"""Host check: the C++ caller of the C ABI compiles against include/eidola_attn.h and links
the library (no GPU needed to build it; tests/test_gpu_cpp_caller.py runs it)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_abi_caller_builds(tmp_path):
    src = os.path.join(ROOT, "tests", "cpp", "abi_caller.cpp")
    lib = os.path.join(ROOT, "eidola_amd", "csrc")
    assert os.path.exists(os.path.join(lib, "libeidola_attn_hip.so")), "build the library first"
    out = tmp_path / "abi_caller"
    subprocess.run(["/opt/rocm/bin/hipcc", "-O1", "-std=c++17", "-x", "c++", "-D__HIP_PLATFORM_AMD__",
                    "-I", os.path.join(ROOT, "include"), "-I/opt/rocm/include", src, "-o", str(out),
                    "-L", lib, "-leidola_attn_hip", "-L/opt/rocm/lib", "-lamdhip64",
                    "-Wl,-rpath," + lib, "-Wl,-rpath,/opt/rocm/lib"], check=True, timeout=300)
    assert os.path.getsize(out) > 0
    # pure C, too: the header is a C header
    c = tmp_path / "c_only.c"
    c.write_text('#include "eidola_attn.h"\n#include "eidola_sched.h"\n'
                 "int main(void) { eid_attn_desc d = {0}; d.struct_size = sizeof d; return (int)d.num_seqs; }\n")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", str(c),
                    "-o", str(tmp_path / "c_only.o")], check=True)
