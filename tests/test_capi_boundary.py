"""The C boundary without a GPU: the library loads, exports every symbol that
include/rocshmem_amd.h declares, the Python binding covers them all, and the
public C++ headers accept the reference's example kernels unchanged."""
import ctypes
import glob
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "rocshmem_amd.h")
PROBES_HEADER = os.path.join(ROOT, "include", "rocshmem_amd_probes.h")
REFERENCE = "/root/reference"


def declared_symbols(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rocshmem_amd_\w+)\s*\(", text)))


def test_header_declares_a_complete_surface():
    names = declared_symbols()
    for needed in ("init", "malloc", "rma", "putmem", "wg_reduce", "to_all", "alltoallmem",
                   "broadcastmem", "amo", "put_signal", "pingpong", "wait_test", "ctx_cycle",
                   "wf_coalesce", "team_split_strided"):
        assert "rocshmem_amd_" + needed in names


def test_library_exports_every_declared_symbol(L):
    lib = ctypes.CDLL(L.LIB_PATH)
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, missing


def test_python_binding_matches_header(L):
    assert sorted(L.SIGNATURES) == declared_symbols()


def test_measuring_probes_live_in_a_library_of_their_own(L):
    """The benchmark's yardsticks are declared in their own header, exported by
    their own library and by nothing in the product's."""
    names = declared_symbols(PROBES_HEADER)
    assert sorted(L.PROBE_SIGNATURES) == names and names
    probes = ctypes.CDLL(L.PROBES_PATH)
    assert not [n for n in names if not hasattr(probes, n)]
    product = ctypes.CDLL(L.LIB_PATH)
    assert not [n for n in names if hasattr(product, n)]
    assert not set(names) & set(declared_symbols())


def test_calls_before_init_fail_cleanly(L):
    l = L.load()
    assert l.set_pe(0) == -1
    assert l.pe_ptr(None, 0) is None
    assert l.rma(L.PUT, L.WG, None, None, 16, 0, 0, 0, 1, 64, 1, None) == -1
    assert l.to_all(L.INT, L.SUM, None, None, 4, 0, 0, 1, None) == -1
    assert l.n_pes() >= 1 and l.my_pe() == 0  # usable before init (src/rocshmem.cpp:113-121)


def test_missing_library_is_an_error_not_a_fallback(L, tmp_path):
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        L.Library(str(tmp_path / "nope.so"))


@pytest.mark.skipif(not os.path.isdir(REFERENCE) or not shutil.which("hipcc"),
                    reason="needs the reference tree and hipcc (build container only)")
@pytest.mark.parametrize("example", ["rocshmem_allreduce_test.cc", "rocshmem_alltoall_test.cc",
                                     "rocshmem_broadcast_test.cc", "rocshmem_getmem_test.cc",
                                     "rocshmem_put_signal_test.cc"])
def test_reference_examples_compile_unchanged(example, tmp_path):
    """Drop-in check of the C++ API: the reference's example programs, read
    from the reference tree where they lie, compile for gfx950 against this
    repository's headers."""
    src = os.path.join(REFERENCE, "examples", example)
    out = tmp_path / (example + ".o")
    cmd = ["hipcc", "--offload-arch=gfx950", "-std=c++17", "-O1", "-x", "hip",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-Wno-unused-command-line-argument",
           "-DROCSHMEM_AMD_NO_MPI_HEADER", "-I", os.path.join(ROOT, "include"), "-c", src,
           "-o", str(out)]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-3000:]
    assert out.exists()


@pytest.mark.skipif(not os.path.isdir(REFERENCE) or not shutil.which("hipcc"),
                    reason="needs the reference tree and hipcc (build container only)")
@pytest.mark.parametrize("extra", [["-mcode-object-version=4"], ["-DUSE_FUNC_CALL"]],
                         ids=["code_object_v4", "real_calls"])
def test_headers_compile_with_an_older_code_object_and_with_real_calls(extra, tmp_path):
    """The public headers read the work-group extents from the implicit kernel
    arguments of code object version 5 and later and fall back to blockDim
    before that; USE_FUNC_CALL keeps the reference's real calls to the device
    API (include/rocshmem/rocshmem_common.hpp in the reference).  Either way a
    reference example compiles for gfx950."""
    src = os.path.join(REFERENCE, "examples", "rocshmem_allreduce_test.cc")
    out = tmp_path / "ex.o"
    cmd = ["hipcc", "--offload-arch=gfx950", "-std=c++17", "-O1", "-x", "hip",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-Wno-unused-command-line-argument", "-DROCSHMEM_AMD_NO_MPI_HEADER", *extra,
           "-I", os.path.join(ROOT, "include"), "-c", src, "-o", str(out)]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-3000:]
    assert out.exists()


@pytest.mark.skipif(not os.path.isdir(REFERENCE) or not shutil.which("hipcc"),
                    reason="needs the reference tree and hipcc (build container only)")
def test_every_function_name_of_the_reference_headers_is_declared(tmp_path):
    """Every rocshmem_* function the reference's public headers declare
    (include/rocshmem/*.hpp, over a thousand once the type tables are stamped
    out) exists under the same name in these headers: the preprocessed device
    pass of <rocshmem/rocshmem.hpp> is searched for each of them."""
    def function_names(text):
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"//.*", "", text)
        return set(re.findall(r"\b(rocshmem_\w+)\s*\(", text))

    wanted = set()
    for path in glob.glob(os.path.join(REFERENCE, "include", "rocshmem", "*.hpp")):
        wanted |= function_names(open(path, errors="ignore").read())
    assert len(wanted) > 1000
    src = tmp_path / "api.hip"
    src.write_text("#include <rocshmem/rocshmem.hpp>\n")
    out = tmp_path / "api.i"
    cmd = ["hipcc", "--offload-arch=gfx950", "-std=c++17", "-DROCSHMEM_AMD_NO_MPI_HEADER", "-I",
           os.path.join(ROOT, "include"), "-E", "--cuda-device-only", str(src), "-o", str(out)]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-3000:]
    have = function_names(out.read_text(errors="ignore"))
    assert not sorted(wanted - have), sorted(wanted - have)[:40]


def test_the_header_is_plain_c_and_the_library_links_from_c(L, tmp_path):
    """The boundary is a C ABI: include/rocshmem_amd.h must compile as C99
    (pedantic) and a C program must link with the library and call it.  The
    calls made here need no GPU: the allocator model (SingleHeap / Pow2Bins,
    src/memory/single_heap.cpp:29-64: 128-byte minimum block, power-of-two
    rounding, alloc(0) -> "nullptr") and the size of the rendezvous file."""
    src = tmp_path / "c_abi.c"
    src.write_text(r'''
#include <stdio.h>
#include "rocshmem_amd.h"
#include "rocshmem_amd_probes.h"
int main(void) {
  void *m = rocshmem_amd_heap_model_create(0x1000000, 1u << 20);
  uint64_t a = rocshmem_amd_heap_model_alloc(m, 1), b = rocshmem_amd_heap_model_alloc(m, 129);
  uint64_t none = rocshmem_amd_heap_model_alloc(m, 0);
  uint64_t used = rocshmem_amd_heap_model_used(m);
  int freed = rocshmem_amd_heap_model_free(m, a);
  rocshmem_amd_heap_model_destroy(m);
  printf("%llu %llu %d %llu %d %d\n", (unsigned long long)a, (unsigned long long)b,
         none == UINT64_MAX, (unsigned long long)used, freed, rocshmem_amd_procs_file_bytes() > 0);
  return rocshmem_amd_n_pes() < 0;
}
''')
    exe = tmp_path / "c_abi"
    libdir = os.path.dirname(L.LIB_PATH)
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"),
                        str(src), "-o", str(exe), "-L", libdir, "-lrocshmem_amd", "-Wl,-rpath," + libdir],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-1500:]
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, (r.stdout, r.stderr[-500:])
    a, b, none, used, freed, has_rdv = r.stdout.split()
    assert (int(a), int(b), none, int(used), has_rdv) == (0, 256, "1", 128 + 256, "1"), r.stdout
    assert int(freed) in (0, 1)
