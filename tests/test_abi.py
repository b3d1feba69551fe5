"""
CPU-side checks of the drop-in boundary: the shared library loads, exports every symbol
declared in include/culsh_amd.h (and nothing in the header is missing from the ctypes
prototypes), reports errors instead of crashing when no GPU is present, and its host-side
seeded parameter generator matches the oracle's definition.
"""

import ctypes as C
import os
import re

import numpy as np
import pytest

from culsh_amd import _lib as L
from oracle import culsh_oracle as o

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "culsh_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(culsh_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = L.load()
    names = header_symbols()
    assert len(names) >= 45
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/culsh_amd.h but not exported"


def test_ctypes_prototypes_cover_the_header():
    assert sorted(L.ALL_SYMBOLS) == header_symbols()


def test_no_python_fallback_when_library_is_missing(monkeypatch, tmp_path):
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "LIB_PATH", str(tmp_path / "missing.so"))
    with pytest.raises(ImportError, match="no CPU fallback"):
        L.load()


def test_errors_are_reported_not_fatal():
    import torch

    if torch.cuda.is_available():
        pytest.skip("needs a machine without a GPU")
    lib = L.load()
    h = C.c_void_p()
    assert lib.culsh_ctx_create(0, C.byref(h)) != L.OK
    assert "hipGetDeviceCount" in L.last_error() or "device" in L.last_error()
    with pytest.raises(RuntimeError):
        L.check(lib.culsh_ctx_create(0, C.byref(h)))
    assert lib.culsh_version().startswith(b"culsh_amd")


def test_null_arguments_are_rejected():
    lib = L.load()
    assert lib.culsh_index_get_meta(None, None) == L.ERR_INVALID
    assert lib.culsh_generate_projection_f32(1, 0, 4, None) == L.ERR_INVALID
    assert "bad argument" in L.last_error()
    lib.culsh_index_free(None)
    lib.culsh_candidates_free(None)
    lib.culsh_ctx_destroy(None)


# ------------------------------------------------------------ host-side seeded generator
def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


@pytest.mark.parametrize("seed", [0, 42, 2**63 - 1, 2**64 - 1])
def test_projection_generator_matches_definition(seed):
    lib = L.load()
    rows, d = 24, 16
    P64 = np.empty(rows * d, dtype=np.float64)
    P32 = np.empty(rows * d, dtype=np.float32)
    assert lib.culsh_generate_projection_f64(seed, rows, d, _ptr(P64)) == L.OK
    assert lib.culsh_generate_projection_f32(seed, rows, d, _ptr(P32)) == L.OK
    exact = o.normal_f64_exact(seed, o.STREAM_PROJECTION, rows * d)   # Python ints + libm
    np.testing.assert_array_equal(P64, exact)
    np.testing.assert_array_equal(P32, exact.astype(np.float32))
    np.testing.assert_allclose(P32, o.generate_random_projections(seed, rows, d).reshape(-1), rtol=2e-7)


@pytest.mark.parametrize("dtype,fn", [(np.float32, "culsh_generate_pslsh_params_f32"),
                                      (np.float64, "culsh_generate_pslsh_params_f64")])
def test_pslsh_generator_matches_definition(dtype, fn):
    lib = L.load()
    rows, d, w, seed = 40, 12, 4, 7
    P = np.empty(rows * d, dtype=dtype)
    b = np.empty(rows, dtype=dtype)
    assert getattr(lib, fn)(seed, rows, d, w, _ptr(P), _ptr(b)) == L.OK
    exact = o.normal_f64_exact(seed, o.STREAM_PROJECTION, rows * d).astype(dtype)
    np.testing.assert_array_equal(P, (exact / dtype(w)).astype(dtype))
    _, b_ref = o.generate_random_projections_biases(seed, rows, d, w, dtype)
    np.testing.assert_array_equal(b, b_ref)        # no libm involved: bit-exact
    assert b.min() > 0 and b.max() <= 1


def test_minhash_generator_matches_definition():
    lib = L.load()
    n = 4096
    A = np.empty(n, dtype=np.uint32)
    B = np.empty(n, dtype=np.uint32)
    assert lib.culsh_generate_minhash_params(123, n, _ptr(A), _ptr(B)) == L.OK
    A_ref, B_ref = o.generate_hash_integers(123, n)
    np.testing.assert_array_equal(A, A_ref)
    np.testing.assert_array_equal(B, B_ref)
    assert A.min() >= 1 and int(A.max()) <= o.MINHASH_PRIME - 1 and int(B.max()) <= o.MINHASH_PRIME - 1
    # the same stream normalised for the other prime of the family; any third value is refused
    p31 = o.MINHASH_PRIME_MERSENNE
    assert lib.culsh_generate_minhash_params_mod(123, n, p31, _ptr(A), _ptr(B)) == L.OK
    A_ref, B_ref = o.generate_hash_integers(123, n, p31)
    np.testing.assert_array_equal(A, A_ref)
    np.testing.assert_array_equal(B, B_ref)
    assert A.min() >= 1 and int(A.max()) <= p31 - 1 and int(B.max()) <= p31 - 1
    assert lib.culsh_generate_minhash_params_mod(123, n, o.MINHASH_PRIME, _ptr(A), _ptr(B)) == L.OK
    np.testing.assert_array_equal(A, o.generate_hash_integers(123, n)[0])
    assert lib.culsh_generate_minhash_params_mod(123, n, 4294967295, _ptr(A), _ptr(B)) != L.OK


def test_header_is_plain_c_and_links_from_a_c_program(tmp_path):
    """The boundary is a C ABI: the header compiles as strict C99 and as C++11, and a C program that
    includes it links against the library and calls it (no device work: version string, and a context
    request for a device that does not exist, which must come back as an error code)."""
    import shutil
    import subprocess

    if not shutil.which("gcc"):
        pytest.skip("no C compiler")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    src = tmp_path / "host.c"
    src.write_text(
        '#include <stdio.h>\n#include <string.h>\n#include "culsh_amd.h"\n'
        "int main(void) {\n"
        "    culsh_ctx* ctx = NULL;\n"
        '    if (strncmp(culsh_version(), "culsh_amd", 9) != 0) return 2;\n'
        "    if (culsh_ctx_create(4096, &ctx) == CULSH_OK) return 3;\n"
        "    if (ctx != NULL) return 4;\n"
        '    if (culsh_last_error() == NULL || strlen(culsh_last_error()) == 0) return 5;\n'
        '    puts("ok");\n    return 0;\n}\n')
    inc = os.path.join(root, "include")
    subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-I", inc, "-c", str(src),
                    "-o", str(tmp_path / "host.o")], check=True)
    subprocess.run(["g++", "-std=c++11", "-Wall", "-Wextra", "-Werror", "-I", inc, "-x", "c++", "-c", str(src),
                    "-o", str(tmp_path / "host_cxx.o")], check=True)
    libdir = os.path.join(root, "culsh_amd")
    exe = tmp_path / "host"
    rocm = "/opt/rocm/lib"
    subprocess.run(["gcc", str(tmp_path / "host.o"), "-L", libdir, "-lculsh_amd", "-L", rocm,
                    "-Wl,-rpath," + libdir, "-Wl,-rpath," + rocm, "-Wl,--allow-shlib-undefined", "-o", str(exe)],
                   check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0 and out.stdout.strip() == "ok", (out.returncode, out.stdout, out.stderr)
