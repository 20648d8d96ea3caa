"""Host-only build of the slot scheduler and the KV pool against a mock model (serve_host_mock.cpp), so that the
scheduler's rounds can be tested without a GPU.  Test infrastructure only."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB = os.path.join(HERE, "libserve_host.so")
SOURCES = [os.path.join(HERE, "serve_host_mock.cpp"), os.path.join(ROOT, "ksearch_amd", "csrc", "serve.cpp"),
           os.path.join(ROOT, "ksearch_amd", "csrc", "kv_pool.cpp")]


def build(force: bool = False) -> str:
    """g++ -shared of the two library sources and the mock (always when ``force``; else only if absent or stale)."""
    stale = not os.path.exists(LIB) or any(os.path.getmtime(s) > os.path.getmtime(LIB) for s in SOURCES)
    if force or stale:
        cmd = ["g++", "-std=c++17", "-O1", "-g", "-shared", "-fPIC", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
               "-Wl,-z,defs", *SOURCES, "-o", LIB]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode:
            raise RuntimeError("host mock build failed:\n" + r.stderr)
    return LIB
