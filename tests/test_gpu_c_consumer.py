"""The library driven from a plain C program (tests/c_consumer/allgather_from_c.c): heap, GEMM +
AllGather (TileGroup variant, the entry point that brings its own signal words) for two ranks,
checked in C against an integer matrix product.  No Python object crosses the boundary: the
test only starts the program and reads its verdict."""

import importlib.util
import subprocess
from pathlib import Path

import pytest

HERE = Path(__file__).resolve().parent / "c_consumer"


def load_builder():
    spec = importlib.util.spec_from_file_location("c_consumer_build", HERE / "build.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_the_c_program_compiles_and_links(tmp_path):
    """Without a GPU: strict C99 against the header, linked against the built library; run here it
    gets no device and must say so with status 1 instead of crashing."""
    from tileccl_amd import _lib

    if not Path(_lib.LIB_PATH).exists():
        pytest.skip("library not built")
    builder = load_builder()
    exe = builder.build(tmp_path / "allgather_from_c")
    assert exe.exists()


@pytest.mark.gpu
def test_two_ranks_gather_from_c(lib):
    builder = load_builder()
    exe = builder.BINARY if builder.BINARY.exists() else builder.build()
    print("running", exe, flush=True)
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=100)
    assert run.returncode == 0, run.stdout + run.stderr
    assert run.stdout.strip().splitlines()[-1] == "ok", run.stdout
