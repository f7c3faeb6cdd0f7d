"""Shared helpers of the GPU parity tests: write a generated model to a
directory, run it through the C-ABI executors, run the same graph JSON through
the CPU oracle, and compare storages."""
import json
import os

import numpy as np

from oracle import oracle as O
from reef_amd import binding as B

# fp32 tolerance of the hot path: 1e-4 relative to the tensor's largest magnitude
REL_TOL = 1e-4


def write_model(g, tmpdir):
    out = os.path.join(str(tmpdir), g.name)
    g.write(out)
    return out


def max_rel_err(got, ref):
    ref = np.asarray(ref, np.float64)
    got = np.asarray(got, np.float64)
    denom = max(np.abs(ref).max(), 1e-30)
    return float(np.abs(got - ref).max() / denom)


def compare_storages(exe, oracle, model, skip_names=("temp_arg",), tol=REL_TOL, what=""):
    """Per-layer parity: every float32 storage written by a kernel."""
    written = set()
    for k in model["kernels"]:
        written.update(k["args"])
    worst = (0.0, None)
    for i in sorted(written):
        s = model["storage"][i]
        if s["stype"] != "float32" or s["name"] in skip_names or s["name"].startswith("p"):
            continue
        got = exe.get_data(i, s["size"])
        ref = oracle.storage[i]
        assert np.isfinite(got).all(), "%s storage %d has non-finite values" % (what, i)
        err = max_rel_err(got, ref)
        if err > worst[0]:
            worst = (err, i)
        assert err <= tol, "%s storage %d (%s): rel err %.3e > %.1e" % (what, i, s["name"], err, tol)
    return worst


def run_both(g, tmpdir, inputs, kind=B.BASE, preemptible=False):
    d = write_model(g, tmpdir)
    model = json.load(open(os.path.join(d, g.name + ".json")))
    exe = B.Executor.from_dir(d, g.name, kind)
    pfile = os.path.join(d, g.name + ".param")
    orc = O.GraphOracle(model, pfile if os.path.exists(pfile) else None)
    for name, arr in inputs.items():
        exe.set_input_checked(name, arr)
        orc.set_input(name, arr)
    if preemptible:
        exe.execute_preemptable()
    else:
        exe.execute()
    orc.run()
    return exe, orc, model
