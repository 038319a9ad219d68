"""What the compiler made of the kernels, checked on the compiled code (no GPU needed).

A select between an LDS read and a read from memory (`c ? lds[i] : mem[j]`), or an address that
was rebuilt from an integer, is compiled to a flat load.  A flat load counts as an access to
memory and to LDS at once, and the wait behind it also waits for every store the wave still has
under way; the merge engine once had one per position.  The library's kernels hold none (one atomic
per k-mer launch apart): this test keeps it so."""
import os
import re
import subprocess

import pytest

from dnatok_amd import build

SOURCES = ["bpe_encode.hip", "kmer_encode.hip", "char_encode.hip", "pack.hip"]


@pytest.mark.parametrize("src", SOURCES)
def test_no_flat_loads_or_stores_in_the_kernels(src, tmp_path):
    hipcc = build.hipcc()
    if not (os.path.isabs(hipcc) and os.path.exists(hipcc)):
        pytest.skip("hipcc not found")
    out = tmp_path / (src + ".s")
    flags = [f for f in build.HIPCC_FLAGS if f not in ("-fPIC",)]
    subprocess.check_call([hipcc, *flags, "-I", build.CSRC, "-S", "--cuda-device-only", "-o", str(out),
                           os.path.join(build.CSRC, src)], stderr=subprocess.DEVNULL)
    bad = []
    kernel = None
    for line in out.read_text().splitlines():
        m = re.match(r"^(_Z\w+):", line)
        if m:
            kernel = m.group(1)
        code = line.split(";")[0]
        if re.search(r"\bflat_(load|store)_", code):
            bad.append((kernel, code.strip()))
    assert not bad, f"{len(bad)} flat loads / stores, e.g. {bad[:3]}"
