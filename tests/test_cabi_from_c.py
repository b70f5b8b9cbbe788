"""The public header as a C consumer sees it: it compiles as strict C99, its struct layouts are
those of the ctypes table (every field's offset and the total size, as gcc lays them out), its
constants are the Python side's, and a plain C program links against the library and gets the
documented status codes back from calls that are rejected on the host (no GPU is touched)."""

import ctypes as C
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
INCLUDE = ROOT / "include"

STRUCTS = {  # header name -> ctypes class
    "tccl_device_info": "DeviceInfo",
    "tccl_gemm_desc": "GemmDesc",
    "tccl_sync_desc": "SyncDesc",
    "tccl_heap_view": "HeapView",
    "tccl_scatter_desc": "ScatterDesc",
    "tccl_transport_desc": "TransportDesc",
    "tccl_static_plan": "StaticPlan",
}
CONSTANTS = {  # header macro / enumerator -> name in tileccl_amd._lib
    "TCCL_ERR_INVALID": "ERR_INVALID",
    "TCCL_ERR_UNSUPPORTED": "ERR_UNSUPPORTED",
    "TCCL_F16": "F16",
    "TCCL_BF16": "BF16",
    "TCCL_F32": "F32",
    "TCCL_GEMM_B_KMAJOR": "GEMM_B_KMAJOR",
    "TCCL_STAGED_ALLREDUCE": "STAGED_ALLREDUCE",
    "TCCL_STAGED_SCATTER": "STAGED_SCATTER",
}

pytestmark = pytest.mark.skipif(shutil.which("gcc") is None, reason="needs gcc")


def build_and_run(tmp_path, body, link=False):
    src = tmp_path / "probe.c"
    src.write_text('#include <stddef.h>\n#include <stdio.h>\n#include <string.h>\n#include "tileccl_hip.h"\n'
                   "int main(void) {\n" + body + "  return 0;\n}\n")
    exe = tmp_path / "probe"
    cmd = ["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", f"-I{INCLUDE}", str(src), "-o", str(exe)]
    if link:
        from tileccl_amd import _lib

        lib = Path(_lib.LIB_PATH)
        if not lib.exists():
            pytest.skip("library not built")
        cmd += [f"-L{lib.parent}", "-ltileccl_hip", f"-Wl,-rpath,{lib.parent}", "-Wl,-rpath,/opt/rocm/lib"]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    return subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout


def test_struct_layouts_as_gcc_sees_them(tmp_path):
    from tileccl_amd import _lib

    body = ""
    for cname, pyname in STRUCTS.items():
        cls = getattr(_lib, pyname)
        body += f'  printf("{cname} size %zu\\n", sizeof({cname}));\n'
        for field, _ in cls._fields_:
            body += f'  printf("{cname} {field} %zu\\n", offsetof({cname}, {field}));\n'
    seen = {}
    for line in build_and_run(tmp_path, body).splitlines():
        cname, field, value = line.split()
        seen[(cname, field)] = int(value)
    for cname, pyname in STRUCTS.items():
        cls = getattr(_lib, pyname)
        assert seen[(cname, "size")] == C.sizeof(cls), cname
        for field, _ in cls._fields_:
            assert seen[(cname, field)] == getattr(cls, field).offset, f"{cname}.{field}"


def test_constants_as_gcc_sees_them(tmp_path):
    from tileccl_amd import _lib

    body = "".join(f'  printf("{c} %d\\n", (int){c});\n' for c in CONSTANTS)
    seen = dict(line.split() for line in build_and_run(tmp_path, body).splitlines())
    for cname, pyname in CONSTANTS.items():
        assert int(seen[cname]) == getattr(_lib, pyname), cname


def test_a_c_program_links_and_is_refused_on_the_host(tmp_path):
    from tileccl_amd import _lib

    body = """
  tccl_gemm_desc d;
  memset(&d, 0, sizeof d);
  printf("abi %d\\n", tccl_abi_version());
  printf("null %d\\n", tccl_gemm(NULL, NULL));
  printf("empty %d\\n", tccl_gemm(&d, NULL));
  printf("text %s\\n", tccl_last_error_string());
"""
    out = dict(line.split(" ", 1) for line in build_and_run(tmp_path, body, link=True).splitlines())
    assert out["abi"] == "1"
    assert int(out["null"]) == _lib.ERR_INVALID and int(out["empty"]) == _lib.ERR_INVALID
    assert out["text"].strip()
