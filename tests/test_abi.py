"""The C ABI library loads without a GPU and exports every symbol include/mmreshard.h declares."""
import ctypes
import os
import re
import subprocess

import pytest

import multimesh_jax_amd as mm
from multimesh_jax_amd import _binding as B

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HAVE_GPU = os.path.exists("/dev/kfd")


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "mmreshard.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mmr_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    lib = ctypes.CDLL(B.LIB_PATH)
    names = _declared_symbols()
    assert len(names) >= 40
    for name in names:
        assert hasattr(lib, name), "libmmreshard.so does not export " + name
        assert name in B.PROTOTYPES, "the ctypes binding does not type " + name
    assert sorted(B.PROTOTYPES) == names


def test_struct_layouts_match_the_header():
    # sizes the C compiler gives the PODs of the header
    src = r'''
    #include <stdio.h>
    #include "mmreshard.h"
    int main(void) {
      printf("%zu %zu %zu %zu %zu %zu %zu\n", sizeof(mmr_sharded_shape), sizeof(mmr_op_sharding), sizeof(mmr_copy_chunk),
             sizeof(mmr_transpose_chunk), sizeof(mmr_plan_options), sizeof(mmr_plan_stats), sizeof(mmr_context_stats));
      return 0;
    }'''
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "s.c")
        open(c, "w").write(src)
        exe = os.path.join(d, "s")
        subprocess.check_call(["gcc", "-std=c11", "-I", os.path.join(ROOT, "include"), c, "-o", exe])
        sizes = [int(x) for x in subprocess.check_output([exe]).split()]
    got = [ctypes.sizeof(t) for t in (B.ShardedShape, B.OpSharding, B.CopyChunk, B.TransposeChunk, B.PlanOptions,
                                      B.PlanStats, B.ContextStats)]
    assert got == sizes


def test_version_and_itemsize():
    lib = mm.load()
    assert b"gfx950" in lib.mmr_version()
    assert [mm.itemsize(t) for t in ("PRED", "BF16", "F32", "C64", "C128", "F8E4M3FN")] == [1, 2, 4, 8, 16, 1]
    assert lib.mmr_itemsize(55) == 0


@pytest.mark.skipif(HAVE_GPU, reason="checks the behaviour on a machine without a GPU")
def test_no_gpu_means_a_loud_error_not_a_fallback():
    with pytest.raises(mm.MmrError) as e:
        mm.ReshardContext(0)
    assert e.value.status_name == "HIP_ERROR"
    assert "no CPU fallback" in str(e.value)


@pytest.mark.skipif(HAVE_GPU, reason="checks the behaviour on a machine without a GPU")
def test_cpp_mirror_fails_loudly_without_gpu():
    exe = os.path.join(ROOT, "tests", "cpp", "hip_execute_context_test")
    if not os.path.exists(exe):
        subprocess.check_call(["bash", os.path.join(ROOT, "tests", "cpp", "build.sh")])
    p = subprocess.run([exe], capture_output=True, text=True)
    assert p.returncode == 2
    assert "no CPU fallback" in p.stderr


@pytest.mark.gpu
def test_cpp_mirror_of_the_execute_context():
    """HipExecuteContext driven like MultiMeshPjRtExecutable::Execute drives the reference context."""
    exe = os.path.join(ROOT, "tests", "cpp", "hip_execute_context_test")
    assert os.path.exists(exe), "build it with tests/cpp/build.sh"
    print("[gpu-test] running " + exe, flush=True)
    p = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stdout + p.stderr
    assert p.stdout.strip().endswith("OK")
