"""The rocprofv3 summaries under profiles/ record the SHA-256 of the kernel source they were taken on; bench.py reports a
workload's HBM traffic from its summary only while the source it emits still has that hash.  This test keeps the two
together: every benchmark workload has a summary, and the summary belongs to the kernel the library emits today."""
import glob
import hashlib
import os
import re

import pytest

from kernelcodegen_amd.configs import WORKLOADS, workload_source

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("name", sorted(WORKLOADS))
def test_profile_summary_belongs_to_the_emitted_kernel(name):
    source, info, family, params = workload_source(name)
    files = glob.glob(os.path.join(ROOT, "profiles", "%s__%s.md" % (family, name)))
    assert len(files) == 1, "no summary profiles/%s__%s.md" % (family, name)
    text = open(files[0]).read()
    sha = re.search(r"^kernel_source_sha256:\s*([0-9a-f]{64})\s*$", text, re.M)
    traffic = re.search(r"^hbm_traffic_bytes:\s*(\d+)\s*$", text, re.M)
    assert sha and traffic, "the summary lacks the two lines bench.py reads"
    assert sha.group(1) == hashlib.sha256(source.encode()).hexdigest(), \
        "the kernel source has changed since the summary was taken: profile the workload again"
    assert "rocprofv3 --kernel-trace --stats" in text and "--workload %s " % name in text
    assert int(traffic.group(1)) > 0
