"""Building a C++ program against the engine's library API (used by CPU and GPU tests)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def build_demo(out_dir) -> str:
    from photon_infer_amd.ops import build

    lib = build.build_module("api", quiet=True)
    cxx = build._host_compiler()
    exe = os.path.join(str(out_dir), "engine_demo")
    cmd = [cxx, "-O1", "-std=c++17", os.path.join(ROOT, "tests", "cpp", "engine_demo.cpp"),
           "-I", os.path.join(build.CSRC_DIR, "api"), "-L", os.path.dirname(lib), "-lphoton_api",
           f"-Wl,-rpath,{os.path.dirname(lib)}", "-o", exe]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr
    return exe


def run_demo(exe, *args, timeout=300):
    env = dict(os.environ, PHOTON_INFER_AMD_ROOT=ROOT)
    return subprocess.run([exe, *[str(a) for a in args]], capture_output=True, text=True, timeout=timeout, env=env)
