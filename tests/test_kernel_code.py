"""A property of the compiled product kernel that its loop relies on and only the compiler's output shows."""

import os
import re
import shutil
import subprocess

import pytest

from mini_llm_amd.csrc import build

HIPCC = shutil.which("hipcc") or ("/opt/rocm/bin/hipcc" if os.path.exists("/opt/rocm/bin/hipcc") else None)


@pytest.mark.skipif(HIPCC is None, reason="no hipcc to compile with")
def test_no_scalar_load_inside_the_loop_of_the_streaming_product(tmp_path):
    # gemm_stream_kernel waits for its fragment reads by count ("at most n LDS operations still under way"), which
    # holds because LDS operations complete in order. Scalar memory loads count on the same counter and complete
    # out of order: one inside the loop (a kernel argument the compiler chose to fetch again there, say) would let
    # such a wait pass with a fragment still on its way. Nothing in the source can forbid that, so the compiled
    # loops are looked at: every loop that holds matrix instructions, in every instantiation.
    listing = tmp_path / "gemm.s"
    subprocess.run([HIPCC, *build.FLAGS, "-S", "--cuda-device-only", "-o", str(listing), str(build.CSRC / "gemm.hip")],
                   check=True, capture_output=True, timeout=600)
    text = listing.read_text()
    kernels = re.split(r"\n(?=_ZN6stream18gemm_stream_kernel[^\n]*:\s)", text)[1:]
    assert len(kernels) >= 11  # five tiles, two output types, and the 256 x 256 tile with bfloat16 out
    for kernel in kernels:
        name = kernel.split(":", 1)[0]
        body = kernel.split(".Lfunc_end", 1)[0].split("\n")
        labels = {m.group(1): i for i, line in enumerate(body) if (m := re.match(r"^(\.LBB\d+_\d+):", line))}
        loops = []
        for i, line in enumerate(body):
            m = re.search(r"s_c?branch\w* (\.LBB\d+_\d+)", line)
            if m and labels.get(m.group(1), i) < i:
                loop = body[labels[m.group(1)] : i + 1]
                if any("v_mfma" in instruction for instruction in loop):
                    loops.append(loop)
        assert loops, name
        for loop in loops:
            scalar_loads = [instruction.strip() for instruction in loop if re.search(r"\ts_(buffer_)?load", instruction)]
            assert not scalar_loads, (name, scalar_loads)
            # and no register of the loop lives in memory
            assert not [instruction for instruction in loop if re.search(r"\tscratch_(load|store)", instruction)], name
        if "Li256ELi256E" in name:
            # the largest tile: 256 sums a lane fill the accumulation registers, and a few values of the prologue (the
            # bias asked for early) wait in memory until the epilogue, outside the loop
            scratch = int(re.search(r"; ScratchSize: (\d+)", kernel).group(1))
            assert scratch <= 64, (name, scratch)
        else:
            assert re.search(r"; ScratchSize: 0\b", kernel), name
