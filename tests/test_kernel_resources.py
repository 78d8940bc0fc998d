"""What the compiler made of the hot kernels: none of them may keep registers in scratch memory
(a spill inside the key loop of the prompt attention kernel once cost a tenth of the prefill
without failing any test), and the blocks that are meant to share a CU must fit it."""
import os
import re
import shutil
import subprocess

import pytest

from sparseengine_amd.kernels import library

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
pytestmark = pytest.mark.skipif(not os.path.exists(HIPCC), reason="no hipcc")

# kernels that may use scratch memory: (source, part of the mangled name) -> bytes per lane
ALLOWED_SCRATCH = {
    ("moe_mfma", "grouped_gemm_mfma_kernelILi2ELi4ELi1ELi2ELi16E"): 64,       # dense product of 33..64 rows, K split 16 ways
    ("moe_mfma", "grouped_gemm_mfma_kernelILi3ELi4ELi1ELi2ELi16E"): 64,       # the same on a tiled copy of the matrix
    # prompt attention at head size 128 on pages that are no multiple of 32 keys: the lanes' own page
    # counters on top of a loop that fills the register file (two or three registers, outside the loop's core)
    ("attention_mfma", "paged_attention_tiled_kernelILi4ELi2ELi4ELb0E"): 16,
}


def resource_usage(name: str, tmp_path) -> dict[str, dict[str, int]]:
    flags = [f for f in library._flags(name) if f not in ("-shared", "-fPIC")]
    proc = subprocess.run([HIPCC, *flags, "-c", "--cuda-device-only", "-Rpass-analysis=kernel-resource-usage",
                           str(library.CSRC / f"{name}.hip"), "-o", str(tmp_path / f"{name}.o")],
                          capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-3000:]
    out = {}
    for block in re.split(r"remark: Function Name: ", proc.stderr)[1:]:
        fields = {key: int(value) for key, value in re.findall(r"remark: +([A-Za-z /\[\]]+?): (\d+)", block)}
        out[block.split(" ")[0]] = fields
    return out


@pytest.mark.parametrize("name", ["attention_mfma", "moe_mfma"])
def test_matrix_core_kernels_keep_their_registers(name, tmp_path):
    usage = resource_usage(name, tmp_path)
    assert usage, "no kernel was reported"
    for kernel, fields in usage.items():
        allowed = max([limit for (source, part), limit in ALLOWED_SCRATCH.items() if source == name and part in kernel] or [0])
        assert fields["ScratchSize [bytes/lane]"] <= allowed, f"{kernel} spills {fields['ScratchSize [bytes/lane]']} bytes per lane"
    if name == "attention_mfma":     # head size 128: two blocks of four wavefronts per CU need two wavefronts per SIMD
        tiled = [f for k, f in usage.items() if "paged_attention_tiled_kernelILi4E" in k]
        assert tiled and all(f["Occupancy [waves/SIMD]"] >= 2 for f in tiled)
    else:                            # the wide expert kernel runs two blocks of eight wavefronts per CU
        wide = [f for k, f in usage.items() if "grouped_gemm_wide_kernel" in k and "Li128ELi32E" in k]
        assert wide and all(f["Occupancy [waves/SIMD]"] >= 4 for f in wide)
