"""The counter summary under profiles/ records the hash of the source file each figure was measured on; bench.py
reports a figure only while that hash matches.  This check fails when a kernel source has changed since its
counters were read, i.e. when the summary has to be regenerated."""
import hashlib
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_traffic_summary_matches_the_kernel_sources():
    text = open(os.path.join(ROOT, "profiles", "hbm_traffic_bench_kernels.md")).read()
    rows = re.findall(r"^\|\s*`(\w+)`\s*\|\s*([\w.-]+)\s*\|\s*([\w./]+)\s*\|\s*([0-9a-f]{16})\s*\|", text, flags=re.M)
    assert rows, "no kernel rows in the summary"
    stale = []
    for kernel, workload, src, digest in rows:
        path = os.path.join(ROOT, "cascading_kv_cache_amd", "csrc", src)
        if hashlib.sha256(open(path, "rb").read()).hexdigest()[:16] != digest:
            stale.append((kernel, workload, src))
    assert not stale, f"counters were read on another version of: {sorted(set(s[2] for s in stale))}"
    # the kernels bench.py asks for
    have = {(k, w) for k, w, _, _ in rows}
    for need in [("fwd_pipe_kernel", "layer64k"), ("decode_stream_kernel", "layer64k"), ("fwd_pipe_kernel", "cfg2"),
                 ("decode_stream_kernel", "cfg3"), ("ckv_update_apply_vec_kernel", "layer64k"),
                 ("ckv_update_one_kernel", "cfg3")]:
        assert need in have, need
