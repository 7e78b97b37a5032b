"""The checked-in inline-asm loops are exactly what their generator writes."""
import os
import subprocess
import sys

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "cudabert_amd", "csrc")


@pytest.mark.parametrize("args,inc", [([], "gemm_bf16_256_loop.inc"), (["half"], "gemm_bf16_256x128_loop.inc")])
def test_inc_matches_generator(args, inc):
    out = subprocess.run([sys.executable, os.path.join(CSRC, "gen_gemm_asm.py")] + args, capture_output=True,
                         text=True, check=True).stdout
    assert out == open(os.path.join(CSRC, inc)).read()
    # the blocks wait for their loads and fragment reads explicitly; every loop has exactly one back edge
    assert out.count("s_cbranch_scc1 L_loop_") == 1 and "s_barrier" in out
