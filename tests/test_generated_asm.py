"""The checked-in inline-asm loops are exactly what their generator writes."""
import os
import subprocess
import sys

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "cudabert_amd", "csrc")


@pytest.mark.parametrize("args,inc", [([], "gemm_bf16_256_loop.inc"), (["half"], "gemm_bf16_256x128_loop.inc"),
                                      (["deep"], "gemm_bf16_256x128_deep_loop.inc"), (["quarter"], "gemm_bf16_128_loop.inc")])
def test_inc_matches_generator(args, inc):
    out = subprocess.run([sys.executable, os.path.join(CSRC, "gen_gemm_asm.py")] + args, capture_output=True,
                         text=True, check=True).stdout
    assert out == open(os.path.join(CSRC, inc)).read()
    # the blocks wait for their loads and fragment reads explicitly; every loop has exactly one back edge
    assert out.count("s_cbranch_scc1 L_loop_") == 1 and "s_barrier" in out


def _written_registers(inc_text):
    """Hard registers (not %[operand] placeholders) that appear as the destination of an
    instruction in a generated loop."""
    import re
    regs = set()
    for line in inc_text.splitlines():
        m = re.match(r'^"\s*([a-z_0-9]+)\s+([^\\]*)\\n"$', line.strip())
        if not m:
            continue
        op, args = m.group(1), m.group(2)
        if op.startswith(("s_waitcnt", "s_barrier", "s_nop", "s_cbranch", "s_cmp", "buffer_load")):
            continue            # no register destination (the loads write LDS)
        dst = args.split(",")[0].strip()
        r = re.match(r"^v\[(\d+):(\d+)\]$", dst)
        if r:
            regs.update("v%d" % i for i in range(int(r.group(1)), int(r.group(2)) + 1))
        elif re.match(r"^(v\d+|s\d+|m0)$", dst):
            regs.add(dst)
        else:
            assert dst.startswith("%["), (op, dst)      # an accumulator operand of the asm statement
    return regs


def _clobbers(hip_text, inc):
    import re
    at = hip_text.index('#include "%s"' % inc)
    stmt = hip_text[at:hip_text.index(");", at)]
    tail = stmt.split(":")[-1]                     # the clobber list is the last section
    regs = set(re.findall(r'"([a-z0-9]+)"', tail))
    for b in re.findall(r"CUBERT_V10\((\d+)\)", tail):
        regs.update("v%s%d" % (b, i) for i in range(10))
    return regs


@pytest.mark.parametrize("inc,hip", [("gemm_bf16_256_loop.inc", "gemm_bf16_256.hip"), ("gemm_bf16_256x128_loop.inc", "gemm_bf16_256.hip"),
                                     ("gemm_bf16_256x128_deep_loop.inc", "gemm_bf16_256.hip"), ("gemm_bf16_128_loop.inc", "gemm_bf16_128.hip")])
def test_every_register_the_loop_writes_is_declared_clobbered(inc, hip):
    written = _written_registers(open(os.path.join(CSRC, inc)).read())
    clob = _clobbers(open(os.path.join(CSRC, hip)).read(), inc)
    assert "m0" in written and "scc" in clob and "memory" in clob
    assert written <= clob, sorted(written - clob)
