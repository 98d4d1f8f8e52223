"""A compile-time property of the one-pass short-range forward kernel, checked on its assembly.

That kernel requests its K and V copies (global -> LDS) first, then its Q, mask and dropout rows,
and waits with `s_waitcnt vmcnt(N)` for the copies alone: loads complete in request order, so once
at most the N loads requested AFTER the copies are outstanding, the copies have landed.  N is
written in the source as the number of those loads; if a compiler ever merged, split, hoisted or
sank one of them the count would be off and the wait too short.  This compiles the kernel's
translation unit to assembly (device side only, no GPU needed) and counts.
"""
import os
import re
import subprocess
import tempfile

import pytest

from nvfuserexamples_amd import build as B

SRC = os.path.join(os.path.dirname(B.__file__), "csrc", "fmha_fwd.hip")
VM_OP = re.compile(r"\s+(global_load|global_store|buffer_load|buffer_store|flat_load|flat_store|scratch_load|scratch_store)")


@pytest.mark.skipif(not os.path.exists(B.HIPCC), reason="needs hipcc")
def test_short_kernel_waits_for_exactly_the_loads_behind_its_copies():
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "fwd.s")
        subprocess.run([B.HIPCC, *B.HIP_FLAGS, "-DFMHA_TU_BF16=0", "-DFMHA_TU_D=64", "-DFMHA_TU_STRIDED=0",
                        "-S", "--cuda-device-only", SRC, "-o", out], check=True, capture_output=True)
        lines = open(out).read().split("\n")
    starts = [i for i, l in enumerate(lines) if re.match(r"^_Z\S*fmha_fwd_short_kernel\S*:", l)]
    # full mask tensor: inference, dropout tensor, dropout tensor + saved outputs; no / per-key mask: without dropout
    # and with the Philox rule; each for any key count and for 97 to 128 keys
    assert len(starts) == 14
    for start in starts:
        end = next(i for i in range(start, len(lines)) if lines[i].startswith(".Lfunc_end"))
        body = lines[start:end]
        copies = [i for i, l in enumerate(body) if "global_load_lds_dwordx4" in l]
        assert copies, lines[start]
        waits = [i for i in range(copies[-1], len(body)) if re.search(r"s_waitcnt vmcnt\(\d+\)", body[i])]
        first = waits[0]
        n = int(re.search(r"vmcnt\((\d+)\)", body[first]).group(1))
        behind = [l for l in body[copies[-1] + 1:first] if VM_OP.match(l)]
        assert n in (4, 12, 20) and len(behind) == n, (lines[start], n, len(behind))   # Q rows (+ mask rows (+ dropout rows))
        # and nothing that reads LDS comes before that wait
        assert not any(re.match(r"\s+ds_read", l) for l in body[:first]), lines[start]
