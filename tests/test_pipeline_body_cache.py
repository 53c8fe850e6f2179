"""CPU: compiled pipeline bodies are kept on disk between processes (DH_PIPELINE_JIT_CACHE, else the user's cache
directory). Each step runs in a process of its own - inside one process a body is compiled once anyway - and compiles
the z-score body without a device (dh_vectorized_pipeline_compile_check)."""
import os
import subprocess
import tempfile
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent

SCRIPT = r"""
import ctypes as C, sys, time
sys.path.insert(0, %r)
from daphne_amd import capi
from daphne_amd.pipeline import KIND_EW_BINARY, KIND_REDUCE_ALL, KIND_ROW_AGG, KIND_STORE_ROW, OPD_ROWVEC, OPD_SCALAR, OPD_SELF, PipeInstr
lib = capi.lib()
lib.dh_vectorized_pipeline_compile_check.argtypes = [C.c_int, C.c_size_t, C.c_int, C.c_void_p, C.c_int]
prog = [PipeInstr(kind=KIND_EW_BINARY, op=1, operand=OPD_ROWVEC, index=0), PipeInstr(kind=KIND_EW_BINARY, op=3, operand=OPD_ROWVEC, index=1),
        PipeInstr(kind=KIND_EW_BINARY, op=2, operand=OPD_SELF), PipeInstr(kind=KIND_ROW_AGG, op=0), PipeInstr(kind=KIND_STORE_ROW, index=0),
        PipeInstr(kind=KIND_EW_BINARY, op=11, domain=1, operand=OPD_SCALAR, scalar=64.0), PipeInstr(kind=KIND_REDUCE_ALL, op=0, domain=1, index=0)]
arr = (PipeInstr * len(prog))(*prog)
t0 = time.perf_counter()
st = lib.dh_vectorized_pipeline_compile_check(0, int(sys.argv[1]), 1, C.cast(arr, C.c_void_p), len(prog))
assert st == capi.DH_OK, lib.dh_last_error().decode()
print("seconds", time.perf_counter() - t0)
""" % str(ROOT)


def compile_in_a_process(env_changes, cols=64):
    env = dict(os.environ)
    env.pop("DH_PIPELINE_JIT_CACHE", None)
    env.update(env_changes)
    # in a directory of its own: with an empty XDG_CACHE_HOME the compiler library keeps a cache below the working directory
    with tempfile.TemporaryDirectory() as cwd:
        r = subprocess.run([sys.executable, "-c", SCRIPT, str(cols)], env=env, cwd=cwd, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    return float(r.stdout.split("seconds")[1])


def test_compiled_bodies_are_found_again_by_the_next_process(tmp_path):
    cache = tmp_path / "bodies"
    first = compile_in_a_process({"DH_PIPELINE_JIT_CACHE": str(cache)})
    files = sorted(cache.iterdir())
    assert len(files) == 1 and files[0].suffix == ".bin" and not list(cache.glob("*.tmp*"))
    blob, stamp = files[0].read_bytes(), files[0].stat().st_mtime_ns
    assert blob[:8] == b"DHJIT001" and b"dh_jit_pipeline" in blob and b"-ffp-contract=off" in blob
    second = compile_in_a_process({"DH_PIPELINE_JIT_CACHE": str(cache)})
    assert sorted(cache.iterdir()) == files and files[0].stat().st_mtime_ns == stamp  # read, not written again
    assert second < first  # no compiler run
    # another body: another file
    compile_in_a_process({"DH_PIPELINE_JIT_CACHE": str(cache)}, cols=32)
    assert len(list(cache.iterdir())) == 2
    # a damaged file is not believed: compiled over, and whole again afterwards
    files[0].write_bytes(blob[: len(blob) // 2])
    compile_in_a_process({"DH_PIPELINE_JIT_CACHE": str(cache)})
    assert files[0].read_bytes() == blob
    files[0].write_bytes(blob.replace(b"-ffp-contract=off", b"-ffp-contract=fast", 1))  # same length, other text
    compile_in_a_process({"DH_PIPELINE_JIT_CACHE": str(cache)})
    assert files[0].read_bytes() == blob


def test_where_the_cache_lives_and_how_it_is_switched_off(tmp_path):
    home, xdg = tmp_path / "home", tmp_path / "xdg"
    home.mkdir()
    compile_in_a_process({"HOME": str(home), "XDG_CACHE_HOME": ""})
    assert len(list((home / ".cache" / "daphne_hip").glob("*.bin"))) == 1
    compile_in_a_process({"HOME": str(home), "XDG_CACHE_HOME": str(xdg)})
    assert len(list((xdg / "daphne_hip").glob("*.bin"))) == 1
    other = tmp_path / "other_home"
    other.mkdir()
    for off in ("off", "0", ""):
        compile_in_a_process({"HOME": str(other), "XDG_CACHE_HOME": "", "DH_PIPELINE_JIT_CACHE": off})
    assert not (other / ".cache").exists()
    # a directory that cannot be made costs nothing but the compilation
    blocked = tmp_path / "a_file"
    blocked.write_text("not a directory")
    compile_in_a_process({"DH_PIPELINE_JIT_CACHE": str(blocked / "below")})
