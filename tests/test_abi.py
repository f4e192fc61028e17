"""The C ABI as a boundary: the built library loads and exports every symbol include/glm53f_kda.h declares, the
header keeps the reference's 13 entry points (crates/glm53f-kda/tests/provenance.rs:41-69), and the ctypes
prototypes agree with the header's parameter counts. No compute call: runs without a GPU."""
import glob
import os
import re
import subprocess

from glm53f_kda import ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declarations():
    text = open(os.path.join(ROOT, "include", "glm53f_kda.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for m in re.finditer(r"\b(?:int|int64_t|const char\*)\s+(glm53f_kda_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        args = m.group(2).strip()
        out[m.group(1)] = 0 if args in ("", "void") else len(args.split(","))
    return out


def test_header_declares_the_reference_entry_points():
    decl = declarations()
    for name in ffi.REFERENCE_SYMBOLS:
        assert name in decl, name
    assert len(ffi.REFERENCE_SYMBOLS) == 13
    extra = set(decl) - set(ffi.REFERENCE_SYMBOLS)
    assert extra == {"glm53f_kda_verify_batch_bf16state", "glm53f_kda_select_batch_bf16state", "glm53f_kda_arch",
                     "glm53f_kda_chain_shift_batch", "glm53f_kda_chain_shift_batch_bf16state", "glm53f_kda_init"}


def test_library_exports_every_declared_symbol():
    lib = ffi.lib()
    decl = declarations()
    assert set(decl) == set(ffi.PROTOTYPES)
    for name, nargs in decl.items():
        assert hasattr(lib, name), name
        assert len(ffi.PROTOTYPES[name][1]) == nargs, name
    assert lib.glm53f_kda_arch() == b"gfx950"


def test_workspace_bytes_is_a_pure_host_function():
    assert ffi.glm53f_kda_prefill_workspace_bytes(64, 1, 2048) == 32 * 148096 * 64
    assert ffi.glm53f_kda_prefill_workspace_bytes(64, 1, 1) == 148096 * 64
    assert ffi.glm53f_kda_prefill_workspace_bytes(0, 1, 16) == 0


def test_the_headers_are_plain_c():
    """The boundary is a C ABI: every header under include/ compiles as C99 on its own, warnings as errors (plain
    pointers and sizes, no C++ and no device-runtime types in the signatures), and a C program that names every
    declared entry point links against the built library."""
    headers = sorted(glob.glob(os.path.join(ROOT, "include", "*.h")))
    assert len(headers) == 3
    for h in headers:
        r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-x", "c", h],
                           capture_output=True, text=True)
        assert r.returncode == 0, r.stderr
    names = []
    for h in headers:
        text = re.sub(r"/\*.*?\*/", "", open(h).read(), flags=re.S)
        names += re.findall(r"\b(glm53f_(?:kda|fwd)_\w+)\s*\(", text)
    names = sorted(set(names))
    assert len(names) == 19 + 2 + 4, names
    prog = "".join(f'#include "{os.path.basename(h)}"\n' for h in headers)
    prog += "int main(void) {\n  const void* p[] = {" + ", ".join(f"(const void*){n}" for n in names) + "};\n"
    prog += "  return p[0] == 0;\n}\n"
    lib_dir = os.path.join(ROOT, "glm53f-afd_amd", "csrc")
    r = subprocess.run(["gcc", "-std=gnu99", "-x", "c", "-", "-I", os.path.join(ROOT, "include"), "-L", lib_dir,
                        "-lglm53f_kda", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath," + lib_dir, "-Wl,-rpath,/opt/rocm/lib",
                        "-o", "/dev/null"], input=prog, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
