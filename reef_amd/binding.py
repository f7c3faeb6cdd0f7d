"""ctypes binding of the flat C API (include/reef_c.h) of libreef_amd.so.

The library is the product; this module only marshals arguments.  It raises if
the library has not been built -- there is no fallback path.
"""
import ctypes
import os

import numpy as np

from .paths import LIB_PATH

STATUS = {0: "Succ", 1: "Fail", 2: "NotFound", 3: "OutOfRange", 4: "Full"}
BASE, TRANS, HYBRID = 0, 1, 2
RUN_DEFAULT, RUN_PREEMPTIBLE = 0, 1

_lib = None


class ReefError(RuntimeError):
    def __init__(self, what, status):
        super().__init__("%s -> %s (%s)" % (what, STATUS.get(status, status), last_error()))
        self.status = status


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libreef_amd.so is not built: run __graft_entry__.build() "
                               "(make -C reef_amd/csrc)")
        # One real-time stream and several best-effort streams have to run side by side; with
        # the runtime's default of 4 hardware queues per process they share queues.  The runtime
        # reads this when it is loaded, so it has to be in the environment before the CDLL call.
        os.environ.setdefault("GPU_MAX_HW_QUEUES", "8")
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.reef_hal_last_error.restype = ctypes.c_char_p
    return _lib


def last_error():
    try:
        return lib().reef_hal_last_error().decode()
    except Exception:  # pragma: no cover
        return ""


def _check(what, st):
    if st != 0:
        raise ReefError(what, st)


def check_model(json_path):
    """(ok, reason): whether every kernel of a graph file fits the storages it names, its operand
    count and its grid -- the check an executor makes when it loads the file, without a device."""
    why = ctypes.create_string_buffer(512)
    st = lib().reef_model_check_kernels(str(json_path).encode(), why, 512)
    return st == 0, why.value.decode()


class Executor:
    """ExecutorBase / TransExecutor / HybridExecutor behind one Python class."""

    def __init__(self, kind=BASE):
        self.kind = kind
        self.h = ctypes.c_void_p()
        _check("create", lib().reef_executor_create(kind, ctypes.byref(self.h)))

    def close(self):
        if self.h:
            lib().reef_executor_destroy(self.h)
            self.h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @classmethod
    def from_dir(cls, model_dir, name, kind=BASE, load_params=True):
        """Loads <dir>/<name>.{json,profile.json,raw.co|trans.co,be.co,param}."""
        e = cls(kind)
        base = os.path.join(model_dir, name)
        if kind == BASE:
            e.load(base + ".json", base + ".raw.co")
        elif kind == TRANS:
            e.load(base + ".json", base + ".trans.co")
        else:
            e.load_hybrid(base + ".json", base + ".profile.json", base + ".trans.co", base + ".be.co")
        if load_params and os.path.exists(base + ".param"):
            e.load_param(base + ".param")
        return e

    def load(self, json_path, co_path):
        _check("load_model_from_file",
               lib().reef_executor_load(self.h, json_path.encode(), co_path.encode()))

    def load_hybrid(self, json_path, profile_path, trans_co, be_co):
        _check("load_hybrid_model_from_file",
               lib().reef_executor_load_hybrid(self.h, json_path.encode(), profile_path.encode(),
                                               trans_co.encode(), be_co.encode()))

    def load_param(self, path):
        _check("load_param_from_file", lib().reef_executor_load_param(self.h, path.encode()))

    def set_input(self, name, arr):
        arr = np.ascontiguousarray(arr)
        return lib().reef_executor_set_input(self.h, name.encode(), arr.ctypes.data_as(ctypes.c_void_p),
                                             ctypes.c_size_t(arr.nbytes))

    def set_input_checked(self, name, arr):
        _check("set_input(%s)" % name, self.set_input(name, arr))

    def get_data_size(self, name):
        sz = ctypes.c_size_t()
        _check("get_data_size", lib().reef_executor_get_data_size(self.h, name.encode(), ctypes.byref(sz)))
        return sz.value

    def get_output(self, n=None):
        if n is None:
            n = self.get_data_size("output") // 4
        out = np.empty(n, np.float32)
        _check("get_output", lib().reef_executor_get_output(self.h, out.ctypes.data_as(ctypes.c_void_p),
                                                           ctypes.c_size_t(out.nbytes)))
        return out

    def get_data(self, idx, n, dtype=np.float32):
        out = np.empty(n, dtype)
        _check("get_data", lib().reef_executor_get_data(self.h, idx, out.ctypes.data_as(ctypes.c_void_p),
                                                       ctypes.c_size_t(out.nbytes)))
        return out

    def set_graph_launch(self, on):
        lib().reef_executor_set_graph_launch(self.h, int(bool(on)))

    def execute(self):
        _check("execute", lib().reef_executor_execute(self.h))

    def execute_to(self, idx):
        _check("execute_to", lib().reef_executor_execute_to(self.h, idx))

    def execute_kernel(self, idx):
        _check("execute_kernel", lib().reef_executor_execute_kernel(self.h, idx))

    def execute_preemptable(self):
        _check("execute_preemptale", lib().reef_executor_execute_preemptable(self.h))

    def num_kernels(self):
        return lib().reef_executor_num_kernels(self.h)

    def poke_preempt_flag(self, value):
        _check("poke_preempt_flag", lib().reef_executor_poke_preempt_flag(self.h, int(value)))

    def read_task_slots(self):
        n = self.num_kernels()
        out = (ctypes.c_int * n)()
        _check("read_task_slots", lib().reef_executor_read_task_slots(self.h, out, n))
        return list(out)

    def kernel_info(self, idx):
        out = (ctypes.c_int * 7)()
        _check("kernel_info", lib().reef_executor_kernel_info(self.h, idx, out))
        keys = ("block_num", "min_occupancy", "vgprs", "sgprs", "lds", "scratch", "op")
        return dict(zip(keys, out))

    def time_kernel(self, idx, flavour=RUN_DEFAULT, warmup=5, iters=50):
        us = ctypes.c_float()
        _check("time_kernel", lib().reef_executor_time_kernel(self.h, idx, flavour, warmup, iters,
                                                             ctypes.byref(us)))
        return us.value

    def time_kernel_dkp_confined(self, idx, layers, task_num, cus, warmup=2, iters=10):
        us = ctypes.c_float()
        _check("time_kernel_dkp_confined", lib().reef_executor_time_kernel_dkp_confined(
            self.h, idx, layers, task_num, cus, warmup, iters, ctypes.byref(us)))
        return us.value

    def time_kernel_in_model(self, idx, flavour=RUN_DEFAULT, samples=5):
        """(in the model's order, directly after itself): one launch between two events, medians."""
        a, b = ctypes.c_float(), ctypes.c_float()
        _check("time_kernel_in_model", lib().reef_executor_time_kernel_in_model(
            self.h, idx, flavour, samples, ctypes.byref(a), ctypes.byref(b)))
        return a.value, b.value

    def time_kernel_dkp_single(self, idx, layers, task_num, cus, evict=None, samples=5):
        us = ctypes.c_float()
        _check("time_kernel_dkp_single", lib().reef_executor_time_kernel_dkp_single(
            self.h, idx, layers, task_num, cus, evict.ptr if evict else None,
            ctypes.c_size_t(evict.nbytes if evict else 0), samples, ctypes.byref(us)))
        return us.value

    def time_kernel_dkp(self, idx, layers, task_num, warmup=2, iters=10):
        us = ctypes.c_float()
        _check("time_kernel_dkp", lib().reef_executor_time_kernel_dkp(self.h, idx, layers, task_num,
                                                                     warmup, iters, ctypes.byref(us)))
        return us.value

    def time_model(self, flavour=RUN_DEFAULT, warmup=5, iters=50):
        lat = (ctypes.c_float * iters)()
        dev = (ctypes.c_float * iters)()
        _check("time_model", lib().reef_executor_time_model(self.h, flavour, warmup, iters, lat, dev))
        return np.array(lat, np.float64), np.array(dev, np.float64)


MODE_NOPREEMPT, MODE_MULTISTREAM, MODE_WAITPREEMPT, MODE_REEF, MODE_RESET = range(5)
QUEUE_RT, QUEUE_BE = 0, 1
STATE_INIT, STATE_WAITING, STATE_EXECUTING, STATE_FINISH = range(4)


class Scheduler:
    """REEFScheduler (src/reef/server/scheduler.h) through the flat C API."""

    def __init__(self, mode=MODE_REEF):
        self.h = ctypes.c_void_p()
        L = lib()
        for fn in ("reef_scheduler_avg_preempt_latency", "reef_scheduler_max_preempt_latency",
                   "reef_scheduler_avg_kernel_sel_latency"):
            getattr(L, fn).restype = ctypes.c_int64
        for fn in ("reef_scheduler_preempt_times", "reef_scheduler_padded_kernels",
                   "reef_scheduler_pending_tasks"):
            getattr(L, fn).restype = ctypes.c_uint64
        L.reef_scheduler_preempt_samples.restype = ctypes.c_size_t
        L.reef_scheduler_preempt_device_samples.restype = ctypes.c_size_t
        L.reef_scheduler_preempt_device_late.restype = ctypes.c_size_t
        L.reef_scheduler_clock_sync_error_ns.restype = ctypes.c_int64
        _check("scheduler_create", L.reef_scheduler_create(mode, ctypes.byref(self.h)))

    def close(self):
        if self.h:
            lib().reef_scheduler_destroy(self.h)
            self.h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def load_model(self, model_dir, name, with_param=True):
        mid = ctypes.c_uint32()
        with_param = with_param and os.path.exists(os.path.join(model_dir, name + ".param"))
        _check("load_model", lib().reef_scheduler_load_model(self.h, model_dir.encode(), name.encode(),
                                                            int(with_param), ctypes.byref(mid)))
        return mid.value

    def create_queue(self, qtype):
        qid = ctypes.c_uint32()
        st = lib().reef_scheduler_create_queue(self.h, qtype, ctypes.byref(qid))
        _check("create_queue", st)
        return qid.value

    def create_queue_status(self, qtype):
        qid = ctypes.c_uint32()
        return lib().reef_scheduler_create_queue(self.h, qtype, ctypes.byref(qid)), qid.value

    def bind_model_queue(self, qid, mid):
        return lib().reef_scheduler_bind_model_queue(self.h, qid, mid)

    def get_data_size(self, mid, name):
        sz = ctypes.c_size_t()
        st = lib().reef_scheduler_get_data_size(self.h, mid, name.encode(), ctypes.byref(sz))
        return st, sz.value

    def set_input(self, mid, arr, name="data"):
        arr = np.ascontiguousarray(arr)
        return lib().reef_scheduler_set_input(self.h, mid, arr.ctypes.data_as(ctypes.c_void_p),
                                              ctypes.c_size_t(arr.nbytes), name.encode())

    def get_output(self, mid, n):
        out = np.empty(n, np.float32)
        _check("get_output", lib().reef_scheduler_get_output(self.h, mid, out.ctypes.data_as(ctypes.c_void_p),
                                                            ctypes.c_size_t(out.nbytes)))
        return out

    def get_data(self, mid, idx, n, dtype=np.float32):
        out = np.empty(n, dtype)
        _check("get_data", lib().reef_scheduler_get_data(self.h, mid, idx, out.ctypes.data_as(ctypes.c_void_p),
                                                        ctypes.c_size_t(out.nbytes)))
        return out

    def new_task(self, mid):
        tid = ctypes.c_uint32()
        _check("new_task", lib().reef_scheduler_new_task(self.h, mid, ctypes.byref(tid)))
        return tid.value

    def new_task_status(self, mid):
        tid = ctypes.c_uint32()
        return lib().reef_scheduler_new_task(self.h, mid, ctypes.byref(tid))

    def wait_task(self, tid):
        return lib().reef_scheduler_wait_task(self.h, tid)

    def task_info(self, tid):
        flags, state = ctypes.c_int(), ctypes.c_int()
        stamps = (ctypes.c_int64 * 3)()
        _check("task_info", lib().reef_scheduler_task_info(self.h, tid, ctypes.byref(flags), stamps,
                                                          ctypes.byref(state)))
        return {"preempted": bool(flags.value & 1), "padded": bool(flags.value & 2),
                "padded_to_complete": bool(flags.value & 4), "submit": stamps[0], "start": stamps[1],
                "end": stamps[2], "state": state.value}

    def run(self):
        _check("run", lib().reef_scheduler_run(self.h))

    def shutdown(self):
        _check("shutdown", lib().reef_scheduler_shutdown(self.h))

    def mode(self):
        return lib().reef_scheduler_mode(self.h)

    def set_wait_sync(self, v):
        lib().reef_scheduler_set_wait_sync(self.h, int(v))

    def set_be_stream_cap(self, v):
        return lib().reef_scheduler_set_be_stream_cap(self.h, int(v))

    def pending_tasks(self):
        return lib().reef_scheduler_pending_tasks(self.h)

    def set_dkp_slack_percent(self, v):
        lib().reef_scheduler_set_dkp_slack_percent(self.h, int(v))

    def avg_preempt_latency(self):
        return lib().reef_scheduler_avg_preempt_latency(self.h)

    def max_preempt_latency(self):
        return lib().reef_scheduler_max_preempt_latency(self.h)

    def avg_kernel_sel_latency(self):
        return lib().reef_scheduler_avg_kernel_sel_latency(self.h)

    def preempt_times(self):
        return lib().reef_scheduler_preempt_times(self.h)

    def padded_kernels(self):
        return lib().reef_scheduler_padded_kernels(self.h)

    def padded_by_op(self):
        """Merged launches by the best-effort side's op id (REEF_OP_* of include/reef_kernels.h)."""
        buf = (ctypes.c_uint64 * 32)()
        n = lib().reef_scheduler_padded_by_op(self.h, buf, 32)
        return [int(buf[i]) for i in range(n)]

    def preempt_samples(self, cap=100000):
        buf = (ctypes.c_int64 * cap)()
        n = lib().reef_scheduler_preempt_samples(self.h, buf, ctypes.c_size_t(cap))
        return np.array(buf[:n], np.int64)

    def preempt_device_samples(self, cap=100000):
        """Preemption latencies measured by the device, in microseconds."""
        buf = (ctypes.c_int64 * cap)()
        n = lib().reef_scheduler_preempt_device_samples(self.h, buf, ctypes.c_size_t(cap))
        return np.array(buf[:n], np.float64) / 1e3

    def preempt_device_late(self, cap=100000):
        """Per device sample: True where a launch reached the device after the flag was raised."""
        buf = (ctypes.c_uint8 * cap)()
        n = lib().reef_scheduler_preempt_device_late(self.h, buf, ctypes.c_size_t(cap))
        return np.array(buf[:n], np.uint8).astype(bool)

    def clock_sync_error_us(self):
        return lib().reef_scheduler_clock_sync_error_ns(self.h) / 1e3

    def preempt_phases(self):
        out = (ctypes.c_int64 * 3)()
        lib().reef_scheduler_preempt_phases(self.h, out)
        return {"flag_ns": out[0], "drop_ns": out[1], "drain_ns": out[2]}

    def run_load(self, rt_mid, be_mids, requests, warmup=0, mean_interval_us=20000.0, seed=0x5EEF,
                 be_only_ms=0):
        """Drives the scheduler with one open-loop real-time client and len(be_mids)
        closed-loop best-effort clients (the request loops of src/example/rpc_client_cont.cpp
        without the RPC hop).  Returns latencies in microseconds and per-client counts."""

        class Cfg(ctypes.Structure):
            _fields_ = [("rt_model", ctypes.c_uint32), ("n_be", ctypes.c_uint32),
                        ("be_models", ctypes.POINTER(ctypes.c_uint32)),
                        ("mean_interval_us", ctypes.c_double), ("seed", ctypes.c_uint64),
                        ("warmup", ctypes.c_int32), ("requests", ctypes.c_int32),
                        ("be_only_ms", ctypes.c_int32)]

        n_be = len(be_mids)
        mids = (ctypes.c_uint32 * max(n_be, 1))(*be_mids)
        cfg = Cfg(rt_mid, n_be, mids, float(mean_interval_us), seed, warmup, requests, be_only_ms)
        lat = np.zeros(requests, np.int64)
        que = np.zeros(requests, np.int64)
        exe = np.zeros(requests, np.int64)
        done = np.zeros(max(n_be, 1), np.uint64)
        pre = np.zeros(max(n_be, 1), np.uint64)
        pad = np.zeros(max(n_be, 1), np.uint64)
        span = ctypes.c_double()
        p = lambda a: a.ctypes.data_as(ctypes.c_void_p)
        _check("loadgen_run", lib().reef_loadgen_run(self.h, ctypes.byref(cfg), p(lat), p(que), p(exe),
                                                     p(done), p(pre), p(pad), ctypes.byref(span)))
        return {"rt_latency_us": lat / 1e3, "rt_queue_us": que / 1e3, "rt_exec_us": exe / 1e3,
                "be_completed": done[:n_be], "be_preempted": pre[:n_be], "be_padded": pad[:n_be],
                "span_s": span.value}


# ---- device memory and the single-convolution entry points ---------------------------------
class DeviceBuffer:
    """Device memory from the C-ABI layer (reef_hal_malloc), for callers of the op-level entry
    points that hold their tensors themselves."""

    def __init__(self, nbytes):
        L = lib()
        _check("hal_init", L.reef_hal_init(0))
        self.ptr = ctypes.c_void_p()
        self.nbytes = int(nbytes)
        _check("hal_malloc", L.reef_hal_malloc(ctypes.c_size_t(max(self.nbytes, 4)), 0, ctypes.byref(self.ptr)))

    @classmethod
    def from_array(cls, arr):
        arr = np.ascontiguousarray(arr)
        b = cls(arr.nbytes)
        _check("h2d", lib().reef_hal_memcpy_h2d(b.ptr, arr.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(arr.nbytes)))
        return b

    def to_array(self, dtype=np.float32):
        out = np.empty(self.nbytes // np.dtype(dtype).itemsize, dtype)
        _check("d2h", lib().reef_hal_memcpy_d2h(out.ctypes.data_as(ctypes.c_void_p), self.ptr, ctypes.c_size_t(out.nbytes)))
        return out

    def fill(self, byte=0):
        _check("memset", lib().reef_hal_memset(self.ptr, int(byte), ctypes.c_size_t(self.nbytes)))

    def free(self):
        if self.ptr:
            lib().reef_hal_free(self.ptr, 0)
            self.ptr = ctypes.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Conv2dDesc(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in ("cin", "h", "w", "cout", "kh", "kw", "stride_h", "stride_w",
                                              "pad_h", "pad_w", "act")]


def ops_init(kernels_co=None):
    from .paths import BUILD_DIR
    path = kernels_co or os.path.join(BUILD_DIR, "reef_kernels.raw.co")
    _check("reef_ops_init", lib().reef_ops_init(path.encode()))


def ops_conv2d(desc, inp, w, bias, residual, out, noalloc=False):
    """reef_ops_conv2d / reef_ops_conv2d_noalloc on DeviceBuffers, default stream; returns the status."""
    fn = lib().reef_ops_conv2d_noalloc if noalloc else lib().reef_ops_conv2d
    st = fn(ctypes.byref(desc), inp.ptr, w.ptr, bias.ptr if bias is not None else None,
            residual.ptr if residual is not None else None, out.ptr, None)
    if st == 0:
        _check("device_sync", lib().reef_hal_device_sync())
    return st
