"""The hand-scheduled kernels must keep what they hold in registers: an accumulator array that the compiler
indexes at run time, or a fragment too many, lands in scratch memory and costs a factor of ten without any
wrong result.  This compiles the sources (no GPU needed) and reads each kernel's private segment size."""
import concurrent.futures
import os
import re
import shutil
import subprocess
import tempfile

import pytest

from tempura_amd.csrc import build

# kernels that must not spill, by a piece of their (mangled) name
NO_SCRATCH = {
    "gemm_pipe.hip": ["gemm_pipe_kernel", "gemm_pipe_big_kernel", "gemm_pipe64_kernel", "gemm_pipe128_kernel"],
    "gemm_mfma.hip": ["gemm_skinny_mfma_kernel", "gemm_skinny_lds_kernel"],
    "attention_mfma.hip": ["attn_prefill_lds_kernel", "attn_decode_kernel"],
    "sampling.hip": ["sample_scale_kernel", "sample_topk_kernel"],      # (keys of a piece, or candidates, in registers)
}


def _private_segment_sizes(source: str, out_dir: str):
    hipcc = build._hipcc()
    asm = os.path.join(out_dir, os.path.basename(source) + ".s")
    subprocess.run([hipcc, *[f for f in build.FLAGS if f != "-fPIC"], "-S", "--cuda-device-only", source, "-o", asm],
                   check=True, capture_output=True)
    sizes = {}
    name = None
    for line in open(asm):
        m = re.match(r"\s*\.amdhsa_kernel\s+(\S+)", line)
        if m:
            name = m.group(1)
        m = re.match(r"\s*\.amdhsa_private_segment_fixed_size\s+(\d+)", line)
        if m and name:
            sizes[name] = int(m.group(1))
    return sizes


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="no hipcc")
def test_hot_kernels_use_no_scratch_memory():
    src_dir = os.path.dirname(build.__file__)
    with tempfile.TemporaryDirectory() as tmp, concurrent.futures.ThreadPoolExecutor(3) as pool:
        jobs = {f: pool.submit(_private_segment_sizes, os.path.join(src_dir, f), tmp) for f in NO_SCRATCH}
        for f, names in NO_SCRATCH.items():
            sizes = jobs[f].result()
            for piece in names:
                found = {k: v for k, v in sizes.items() if piece in k}
                assert found, f"{f}: no kernel named like {piece}"
                spilled = {k: v for k, v in found.items() if v != 0}
                assert not spilled, f"{f}: kernels with scratch memory: {spilled}"
