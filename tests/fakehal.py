"""Python side of the recording backend (tests/fake_hal): installs it into
libreef_amd.so and runs every completed "kernel" with the CPU oracle, decoding
the packed kernel arguments exactly as the gfx950 kernels do
(include/reef_kernels.h).  Test infrastructure only."""
import ctypes
import os
import subprocess

import numpy as np

from oracle import oracle as O
from reef_amd import binding as B

HERE = os.path.dirname(os.path.abspath(__file__))
SO = os.path.join(HERE, "fake_hal", "libreef_fakehal.so")


class OpDesc(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p * 10), ("attr", ctypes.c_int32 * 24)]


class BeArg(ctypes.Structure):
    # ReefBeArgs of include/reef_kernels.h: the C-ABI layer's completion record comes first
    _fields_ = [("done_word", ctypes.c_void_p), ("exit_ticks", ctypes.c_void_p), ("exit_count", ctypes.c_void_p),
                ("seq", ctypes.c_uint32), ("reserved", ctypes.c_uint32),
                ("preempted", ctypes.c_void_p), ("task_slot", ctypes.c_void_p), ("desc", OpDesc)]


class DkpSide(ctypes.Structure):
    _fields_ = [("op", ctypes.c_int32), ("layers", ctypes.c_int32), ("task_num", ctypes.c_int32),
                ("task_offset", ctypes.c_int32), ("desc", OpDesc)]


class DkpArgs(ctypes.Structure):
    _fields_ = [("l", DkpSide), ("r", DkpSide), ("cu_partition", ctypes.c_int32),
                ("num_cus", ctypes.c_int32), ("num_xcds", ctypes.c_int32), ("reserved", ctypes.c_int32),
                ("task_slot_r", ctypes.c_void_p), ("entry_l", ctypes.c_void_p), ("entry_r", ctypes.c_void_p)]


class DeviceInfo(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in ("num_cus", "num_xcds", "simds_per_cu", "max_waves_per_simd",
                                            "vgprs_per_simd", "vgpr_granule", "lds_bytes_per_cu",
                                            "lds_granule", "max_wg_per_cu", "max_threads_per_cu",
                                            "clock_khz")] + \
               [("arch", ctypes.c_char * 32)]


OP_SYMBOL = {1: "reef_conv2d", 2: "reef_splitk_reduce", 3: "reef_dwconv2d", 4: "reef_pool2d",
             5: "reef_global_avgpool", 6: "reef_eltwise", 7: "reef_dense", 8: "reef_softmax",
             9: "reef_layernorm", 10: "reef_bias_gelu", 11: "reef_embedding", 12: "reef_copy",
             13: "reef_transpose", 14: "reef_gemm", 15: "add", 16: "multiply", 17: "reef_attention"}

CB_TYPE = ctypes.CFUNCTYPE(None, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_void_p, ctypes.c_size_t,
                           ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint32),
                           ctypes.c_uint32, ctypes.c_int)


class FakeHal:
    def __init__(self):
        deps = [os.path.join(HERE, "fake_hal", "fake_hal.cpp"),
                os.path.join(os.path.dirname(HERE), "include", "reef_hal.h")]   # the backend table's layout
        if not os.path.exists(SO) or os.path.getmtime(SO) < max(os.path.getmtime(d) for d in deps):
            subprocess.check_call(["make", "-B", "-C", os.path.join(HERE, "fake_hal")],
                                  stdout=subprocess.DEVNULL)
        self.core = B.lib()
        self.lib = ctypes.CDLL(SO)
        self.lib.fake_hal_backend.restype = ctypes.c_void_p
        self.lib.fake_hal_extent.restype = ctypes.c_size_t
        self.lib.fake_hal_extent.argtypes = [ctypes.c_void_p]
        for f in ("fake_hal_launches", "fake_hal_completed", "fake_hal_dropped", "fake_hal_log_size",
                  "fake_hal_graph_launches"):
            getattr(self.lib, f).restype = ctypes.c_long
        self.events = []          # (symbol, flavour, stream, grid, skipped)
        self.skipped = 0
        self._cb = CB_TYPE(self._on_kernel)

    # -- install / remove --------------------------------------------------------
    def install(self, num_cus=256, num_xcds=8, gfx906=False):
        self.lib.fake_hal_reset()
        info = DeviceInfo()
        if gfx906:   # the reference's part (src/reef/executor/hip/hip_impl.cpp:55-74)
            vals = (num_cus, num_xcds, 4, 10, 256, 4, 64 * 1024, 256, 40, 2048, 1725000)
        else:
            vals = (num_cus, num_xcds, 4, 8, 512, 8, 160 * 1024, 1280, 32, 2048, 2400000)
        for (n, _), v in zip(DeviceInfo._fields_[:11], vals):
            setattr(info, n, v)
        info.arch = b"fake"
        self.lib.fake_hal_set_device(ctypes.byref(info))
        self.lib.fake_hal_set_callback(self._cb)
        self.core.reef_hal_set_backend(ctypes.c_void_p(self.lib.fake_hal_backend()))
        self.core.reef_gpuconfig_override_geometry(num_cus, num_xcds)
        self.events.clear()
        self.skipped = 0
        return self

    def remove(self):
        # objects created on this backend must be destroyed on it
        import gc
        gc.collect()
        self.core.reef_hal_set_backend(None)
        self.core.reef_gpuconfig_override_geometry(0, 0)
        self.lib.fake_hal_set_callback(ctypes.cast(None, CB_TYPE))

    def set_kernel_resource(self, name, lds=0, vgprs=32, sgprs=16, stack=0):
        self.lib.fake_hal_set_kernel_resource(name.encode(), lds, vgprs, sgprs, stack)

    def set_missing(self, name):
        self.lib.fake_hal_set_missing(name.encode())

    def log(self):
        out = []
        buf = ctypes.create_string_buffer(128)
        st, g, b, l = ctypes.c_int(), ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint32()
        for i in range(self.lib.fake_hal_log_size()):
            self.lib.fake_hal_log_entry(ctypes.c_long(i), buf, ctypes.c_size_t(128), ctypes.byref(st),
                                        ctypes.byref(g), ctypes.byref(b), ctypes.byref(l))
            out.append((buf.value.decode(), st.value, g.value, b.value, l.value))
        return out

    # -- kernel execution on the CPU ---------------------------------------------
    def _view(self, ptr, dtype=np.float32):
        n = self.lib.fake_hal_extent(ptr)
        if not ptr or n == 0:
            return np.zeros(0, dtype)
        return np.frombuffer((ctypes.c_char * n).from_address(ptr), dtype=dtype)

    def _run_desc(self, symbol, desc, blocks, first=0, count=None):
        """Applies one kernel's effect.  `first`/`count` select a task range (DKP pieces):
        mocked kernels are applied per task, everything else when its last task runs."""
        attrs = list(desc.attr)
        if symbol in ("add", "multiply"):
            a, b, out = (self._view(desc.ptr[i]) for i in range(3))
            count = 64 if count is None else count
            for t in range(first, first + count):
                sl = slice(t * 128, (t + 1) * 128)
                out[sl] = a[:128] * b[sl] if symbol == "multiply" else a[:128] + b[sl]
            return
        total = blocks
        if count is not None and first + count < total:
            return   # an earlier piece of a split launch: the last piece applies the kernel
        views = []
        for i in range(10):
            dt = np.int64 if (symbol == "reef_embedding" and i == 0) else np.float32
            views.append(self._view(desc.ptr[i], dt))
        orc = O.GraphOracle.__new__(O.GraphOracle)
        orc.storage = views
        orc.model = {}
        orc.run_kernel({"name": symbol, "attrs": attrs, "args": list(range(10)),
                        "launch_params": [blocks, 1, 1, 256, 1, 1]})

    def _on_kernel(self, symbol, module_path, kernarg, nbytes, grid, block, lds, stream):
        symbol = symbol.decode()
        path = module_path.decode()
        flavour = "be" if path.endswith(".be.co") else "trans" if path.endswith(".trans.co") else "raw"
        nblocks = grid[0] * grid[1] * grid[2]
        if flavour == "raw":
            d = OpDesc.from_address(kernarg)
            self._run_desc(symbol, d, nblocks)
            self.events.append((symbol, flavour, stream, nblocks, False))
        elif flavour == "be":
            a = BeArg.from_address(kernarg)
            flag = ctypes.c_int32.from_address(a.preempted).value
            if flag:
                self.skipped += 1
                self.events.append((symbol, flavour, stream, nblocks, True))
                return
            self._run_desc(symbol, a.desc, nblocks)
            slot = ctypes.c_int32.from_address(a.task_slot)
            slot.value += nblocks
            self.events.append((symbol, flavour, stream, nblocks, False))
        else:
            a = DkpArgs.from_address(kernarg)
            for side, name in ((a.l, "l"), (a.r, "r")):
                if side.task_num <= 0:
                    continue
                if name == "r" and a.cu_partition >= a.num_cus:
                    continue
                sym = OP_SYMBOL[side.op]
                total = self._total_tasks(sym, side)
                self._run_desc(sym, side.desc, total, side.task_offset, side.task_num)
            self.events.append((symbol, flavour, stream, nblocks, False))

    @staticmethod
    def _total_tasks(sym, side):
        at = side.desc.attr
        if sym in ("add", "multiply"):
            return 64
        if sym == "reef_conv2d":
            return at[15] * at[17] * at[18]
        return side.task_offset + side.task_num
