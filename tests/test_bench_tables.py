"""bench.py's table of profiled HBM traffic must agree with the profile files it names."""
import os
import re

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _profile_figures(path):
    """(kernel name, 'HBM traffic per dispatch: ... = X MB' in bytes) for every kernel block of a profile."""
    out, kernel = [], None
    for line in open(os.path.join(ROOT, path)):
        m = re.match(r"^(w34::\S+|\S+_kernel\S*)", line)
        if m:
            kernel = m.group(1)
        m = re.search(r"HBM traffic per dispatch:.*?=\s*([0-9.]+)\s*MB", line)
        if m:
            out.append((kernel or "", float(m.group(1)) * 1e6))
    return out


def test_profiled_traffic_entries_match_their_profiles():
    assert bench.PROFILED_TRAFFIC
    for workload, (nbytes, path) in bench.PROFILED_TRAFFIC.items():
        assert os.path.exists(os.path.join(ROOT, path)), "%s names a missing profile %s" % (workload, path)
        figs = _profile_figures(path)
        assert figs, "no traffic figure in %s" % path
        # one kernel's figure (the dominant kernel), or, for paths of several kernels, the sum over
        # everything but the append kernel that only fills the pools
        path_sum = sum(f for k, f in figs if "kv_append_kernel" not in k)
        candidates = [f for _, f in figs] + [path_sum]
        assert any(abs(nbytes - f) <= 0.006e6 + 1e-4 * f for f in candidates), (
            "%s: table says %d bytes, %s holds %s" % (workload, nbytes, path, [(k[:30], round(f / 1e6, 2)) for k, f in figs]))
