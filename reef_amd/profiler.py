"""Per-kernel latency profiles for a model directory, measured on the device.

``<model>.profile.json`` drives dynamic kernel padding: ``total_latency`` is the
solo duration of a kernel call and ``latency[j]`` the duration of one round of
``(j + 1) * num_cus`` workgroups, i.e. at occupancy ``j + 1``
(consumed in src/reef/server/scheduler.cpp:509,565-572,589-590).  The reference
ships profiles made by a ``profiler`` binary that is not in its repository
(resource/Makefile:32-36); this module is the equivalent for gfx950.
``total_latency`` / ``latency`` are integer microseconds, at least 1, as the reference's files
hold them; ``total_latency_ns`` / ``latency_ns`` carry the same measurements in nanoseconds
(extra keys the reference's reader does not look up): kernels run for 3-15 us on this device,
so whole microseconds cannot tell which best-effort kernel fits beside which real-time kernel.
"""
import json
import math
import os

from . import binding as B


# larger than the device's last-level cache (256 MiB): overwriting it leaves no operand cached
EVICT_BYTES = 768 << 20


def measure_profile(model_dir, name, iters=10, warmup=2, levels=8, cold=True):
    """cold: add to every figure what the kernel loses when its operands come from HBM instead of
    the caches (one launch between two events after the caches were overwritten, minus the same
    after a launch of the kernel itself).  Back-to-back repetitions of one kernel -- what the
    figures are otherwise made of -- find weights and activations cached; a kernel of a model
    that takes turns with other models does not."""
    exe = B.Executor.from_dir(model_dir, name, B.HYBRID)
    evict = B.DeviceBuffer(EVICT_BYTES) if cold else None
    num_cus = B.lib().reef_gpuconfig_num_cus()
    model = json.load(open(os.path.join(model_dir, name + ".json")))
    kl = {}
    for i, k in enumerate(model["kernels"]):
        info = exe.kernel_info(i)
        blocks = info["block_num"]
        total = exe.time_kernel_dkp(i, info["min_occupancy"], blocks, warmup, iters)
        extra = 0.0
        if cold:
            extra = max(0.0, exe.time_kernel_dkp_single(i, info["min_occupancy"], blocks, 0, evict, 5)
                        - exe.time_kernel_dkp_single(i, info["min_occupancy"], blocks, 0, None, 5))
            total += extra
        max_occ = B.lib().reef_gpuconfig_calculate_occupancy(info["lds"], info["vgprs"], info["sgprs"],
                                                             info["scratch"], 256)
        # latency[j]: one round at occupancy j + 1, with the kernel confined to a few CUs as the
        # best-effort side of a padded launch is, so that j + 1 workgroups really share a CU (on
        # the whole device most kernels do not have the workgroups to reach occupancy 2, and the
        # cost of sharing a CU -- what a CU can pull from memory -- would not show)
        lat = []
        n_levels = min(levels, max(max_occ, 1))
        for j in range(n_levels):
            cus = next((c for c in (32, 16, 8) if (j + 1) * c <= blocks), 0)
            if cus == 0:
                # not enough workgroups for this occupancy even on 8 CUs: it cannot occur
                lat += [lat[-1] if lat else max(1, int(round(total * 1000)))] * (n_levels - len(lat))
                break
            us = exe.time_kernel_dkp_confined(i, j + 1, (j + 1) * cus, cus, warmup, iters)
            lat.append(max(1, int(round((us + extra) * 1000))))
        e = kl.setdefault(k["name"], {"total_latency": 0, "latency": [], "total_latency_ns": 0, "latency_ns": lat})
        e["total_latency_ns"] = max(e["total_latency_ns"], max(1, int(round(total * 1000))))
        e["latency_ns"] = [max(a, b) for a, b in zip(e["latency_ns"], lat)]
        e["total_latency"] = max(1, -(-e["total_latency_ns"] // 1000))
        e["latency"] = [max(1, -(-v // 1000)) for v in e["latency_ns"]]
    lat_us, _ = exe.time_model(B.RUN_DEFAULT, 3, 10)
    prof = {"model_latency": int(math.ceil(float(lat_us.mean()))), "kernel_latency": kl}
    exe.close()
    if evict is not None:
        evict.free()
    return prof


def write_profile(model_dir, name, **kw):
    prof = measure_profile(model_dir, name, **kw)
    with open(os.path.join(model_dir, name + ".profile.json"), "w") as f:
        json.dump(prof, f, separators=(",", ":"))
    return prof
