"""The programs at the repository root, as far as they can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*argv):
    return subprocess.run([sys.executable, *argv], cwd=ROOT, capture_output=True, text=True, timeout=120)


def test_bench_refuses_more_than_one_gpu_with_one_line():
    r = run("bench.py", "--gpus", "2", "--steps", "1", "--warmup", "0")
    assert r.returncode == 2
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


def test_programs_describe_their_options():
    for prog, words in (("bin/trace_run", ["--model", "--dtype", "--out", "--max-tokens"]),
                        ("bin/llama_infer", ["--max-new-tokens", "--temperature", "--dtype"])):
        r = run(prog, "--help")
        assert r.returncode == 0, r.stderr
        for w in words:
            assert w in r.stdout, (prog, w)


def test_graft_entry_has_build_and_smoke():
    sys.path.insert(0, ROOT)
    try:
        import __graft_entry__ as entry
    finally:
        sys.path.pop(0)
    assert callable(entry.build) and callable(entry.smoke)


def test_cpp_program_reports_a_missing_model_folder(tmp_path):
    """The library API for C++ programs builds, links and turns an engine error into an exception."""
    import cpp_api

    exe = cpp_api.build_demo(tmp_path)
    r = cpp_api.run_demo(exe, tmp_path / "no_such_model", "float32", "1,2,3", 4)
    assert r.returncode == 3, (r.stdout, r.stderr)
    # without a GPU the engine refuses before it looks at the folder; with one it names the folder
    assert "engine error:" in r.stderr and ("no_such_model" in r.stderr or "GPU" in r.stderr)
