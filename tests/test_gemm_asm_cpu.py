"""Reads the compiler's assembly of the one-wave-per-SIMD GEMM (ug_amd/csrc/ughip/gemm_dma.hip) on the CPU: the kernel
writes M0 in one inline-asm statement and issues the LDS-writing load that consumes it in another, with an MFMA between
them as the wait state.  No constraint can tell the compiler about that read of M0, so this test holds every build to it:
each global_load_lds_dwordx4 is fed by our own write of M0 and nothing else mentions M0 in between."""
import os
import re
import shutil
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _device_asm():
    from ug_amd import build as b
    hipcc = os.path.join(b.ROCM, "bin", "hipcc")
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc on this box")
    src = os.path.join(b.CSRC, "ughip", "gemm_dma.hip")
    tmp = tempfile.mkdtemp()
    try:
        out = os.path.join(tmp, "gemm_dma.s")
        subprocess.run([hipcc] + b.HIP_FLAGS + ["-w", "--cuda-device-only", "-S", "-I" + b.INC, "-I" + os.path.dirname(src), src, "-o", out],
                       check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
        return open(out).read()
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_every_lds_dma_is_fed_by_the_kernels_own_write_of_m0():
    text = _device_asm()
    kernels = re.findall(r"^(_ZN5ughip\S*gemm_dma4\S*):[^\n]*\n(.*?)^\.Lfunc_end", text, flags=re.S | re.M)
    assert len(kernels) >= 12, len(kernels)
    for name, body in kernels:
        ins = [l.split(";")[0].strip() for l in body.splitlines()]
        ins = [l for l in ins if l and not l.startswith((".", "//")) and not l.endswith(":")]
        pending, mfmas, n_dma = None, 0, 0
        for i, l in enumerate(ins):
            op = l.split()[0]
            if op == "global_load_lds_dwordx4":
                n_dma += 1
                if pending == "add":   # the write needs a wait state before the load: the MFMA(s) the source puts there
                    assert mfmas >= 1, f"{name}: {mfmas} MFMAs between the write of M0 and its load (instruction {i})"
                else:
                    assert pending == "mov" and ins[i - 1].startswith("s_nop") and ins[i - 2].startswith("s_mov_b32 m0"), f"{name}: a load with no write of M0 in front (instruction {i})"
                pending = None
                continue
            if re.search(r"\bm0\b", l):
                assert pending is None, f"{name}: M0 mentioned between a write and its load: {l}"
                assert op in ("s_add_u32", "s_mov_b32") and l.split()[1].rstrip(",") == "m0", f"{name}: unexpected use of M0: {l}"
                pending, mfmas = ("add" if op == "s_add_u32" else "mov"), 0
                continue
            if op.startswith("v_mfma") and pending:
                mfmas += 1
            assert not (pending and op in ("s_cbranch_scc0", "s_cbranch_scc1", "s_branch", "s_barrier", "s_setpc_b64")) or op == "s_barrier", f"{name}: control flow between a write of M0 and its load"
        assert pending is None and n_dma >= 16, (name, n_dma)
