"""Integer logic of the REEF hot path restated from the reference, in plain
Python -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Each function cites the reference lines it follows.  Pinned by: brute force
over small parameter ranges (every task index visited exactly once), closed
forms on hand-computed cases in tests/test_dkp_arithmetic.py, and the
reference's own mocked profile (resource/mocked_kernel/mocked_kernel.profile.json).
"""


def align_up(v, a):
    """src/reef/util/common.h:54-58"""
    r = v % a
    return v if r == 0 else v - r + a


def calculate_occupancy_gfx906(shared_memory, vgprs, sgprs, block_threads):
    """GPUConfig::calculate_occupancy, src/reef/executor/hip/hip_impl.cpp:55-74 (as written,
    including the LDS term that divides by the block size)."""
    vgprs = align_up(vgprs, 4)
    sgprs = align_up(sgprs, 8)
    block_size = align_up(block_threads, 64)
    max_gpr_waves = (16 * 1024 // (vgprs * 64)) * 4
    max_gpr_waves = min(max_gpr_waves, (800 // sgprs) * 4)
    max_gpr_waves = min(max_gpr_waves, 40)
    max_gpr_blocks = max_gpr_waves * 64 // block_size
    max_shared_mem_blocks = 64 * 1024 // block_size
    max_thread_blocks = 2048 // block_size
    return min(max_gpr_blocks, max_shared_mem_blocks, max_thread_blocks)


def logical_layers(block_num, num_cus):
    """src/reef/server/scheduler.cpp:524-525; trans_executor.cpp:138"""
    return align_up(block_num, num_cus) // num_cus


def min_occupancy(block_num, num_cus, max_layers):
    """src/reef/executor/trans_executor.cpp:91-97"""
    return min(logical_layers(block_num, num_cus), max_layers)


def cu_partition(block_num, num_cus):
    """src/reef/server/scheduler.cpp:578; trans_executor.cpp:139-140"""
    layers = logical_layers(block_num, num_cus)
    return align_up(block_num, layers) // layers


def proxy_occupancy_class_gfx906(vgprs, sgprs):
    """TransExecutor::get_proxy_kernel, src/reef/executor/trans_executor.cpp:175-199"""
    sgpr_bound = [102] * 8 + [88, 80]
    vgpr_bound = [256, 128, 84, 64, 48, 40, 36, 32, 28, 28]
    occupancy = 10
    for i in range(1, 10):
        if vgprs > vgpr_bound[i] or sgprs > sgpr_bound[i]:
            occupancy = i
            break
    return occupancy


def device_walk_flat(block_idx, num_cus, part, layers_l, num_l, off_l, layers_r, num_r, off_r):
    """The persistent loop of a transformed kernel, script/generate_asm_loop.py:227-321 and
    its C rendering script/transform_kernel.py:423-478: returns (side, [task indices])."""
    cu_id = block_idx % num_cus
    if cu_id < part:
        side, layers, task_num, task_offset, lower, upper = 0, layers_l, num_l, off_l, 0, part
    else:
        side, layers, task_num, task_offset, lower, upper = 1, layers_r, num_r, off_r, part, num_cus
    layer_idx = block_idx // num_cus
    if layer_idx >= layers:
        return side, []
    idx = (upper - lower) * layer_idx + (cu_id - lower) + task_offset
    step = layers * (upper - lower)
    total = task_offset + task_num
    tasks = []
    while idx < total:
        tasks.append(idx)
        idx += step
    return side, tasks


def decide_padding(rt, be, be_block_offset, num_cus, occupancy_fn):
    """REEFScheduler::dynamic_kernel_padding, the per-kernel decision,
    src/reef/server/scheduler.cpp:533-602.  rt/be are dicts with block_num,
    min_occupancy, threads, vgprs, sgprs, lds, total_latency (+ be['latency'])."""
    merged_block = max(rt["threads"], be["threads"])
    res = dict(vgprs=max(rt["vgprs"], be["vgprs"]), sgprs=max(rt["sgprs"], be["sgprs"]),
               lds=max(rt["lds"], be["lds"]))
    merged_occupancy = occupancy_fn(res["lds"], res["vgprs"], res["sgprs"], merged_block)
    out = dict(merge=False, be_occupancy=0, final_occupancy=rt["min_occupancy"],
               cu_partition=num_cus, be_block_num=0)
    if merged_occupancy < rt["min_occupancy"]:
        return out
    be_occupancy = 0
    for j in range(merged_occupancy - 1, -1, -1):
        if len(be["latency"]) <= j:
            continue
        if be["latency"][j] <= rt["total_latency"]:
            be_occupancy = j + 1
            break
    if be_occupancy == 0:
        return out
    part = cu_partition(rt["block_num"], num_cus)
    be_iters = rt["total_latency"] // be["latency"][be_occupancy - 1]
    n = (num_cus - part) * be_iters * be_occupancy
    if n + be_block_offset > be["block_num"]:
        n = be["block_num"] - be_block_offset
    out.update(merge=True, be_occupancy=be_occupancy,
               final_occupancy=max(rt["min_occupancy"], be_occupancy), cu_partition=part,
               be_block_num=n)
    return out


def rollback(launch_offset, dropped, window, kernel_offset):
    """src/reef/server/scheduler.cpp:320-323"""
    return max(launch_offset - dropped - window, kernel_offset)


def be_kernel_offset(finished, block_nums, begin):
    """HybridExecutor::get_be_kernel_offset, src/reef/executor/hybrid_executor.cpp:141-151"""
    for i in range(begin, len(block_nums)):
        if finished[i] < block_nums[i]:
            return i
    return len(block_nums)
