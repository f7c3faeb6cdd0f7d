"""The reference's RPC front-end, wire-compatible, over the flat C API.

`package reef.rpc; service REEFService` (src/reef/protos/reef.proto:3-79): six unary calls on an
insecure channel, default address `localhost:34543` (src/reef/util/common.h:8).  Control goes over
gRPC, tensors through POSIX shared memory named "<mid>_<name>" (src/reef/server/server.cpp:104,112;
src/reef/util/shared_memory.cpp:13-34), so the reference's own `reef_client` / `reef_client_cont`
binaries talk to this server unchanged.

The image has the gRPC runtime for Python but no protoc and no gRPC for C++, so the messages are
described by hand (one FileDescriptorProto, the classes come from protobuf's message factory) and
the handlers call the scheduler through `include/reef_c.h` exactly as the reference's handlers call
REEFScheduler:

    SetPriority   -> create_queue(RT or BE)                           server.cpp:34-55
    LoadModel     -> load_model(dir/name.{trans.co,be.co,json,profile.json[,param]}) + bind_model_queue   :57-93
    RegisterBlob  -> get_data_size + shared memory "<mid>_<name>"     :95-121
    SetBlob       -> shared memory -> set_input                       :147-169
    GetBlob       -> get_output -> shared memory (always the `output` storage, scheduler.cpp:226-230)   :123-145
    Infer         -> new_task + wait_task                             :171-188

A failing call answers succ = false with gRPC status OK, as the reference does.

Also here: REEFClient / ModelHandle, the Python mirror of src/reef/client/client.cpp:19-141, and
the three command lines of src/example (`python -m reef_amd.rpc server|client|client_cont ...`).
"""
import ctypes
import hashlib
import json
import mmap
import os
import shutil
import sys
import tempfile
import threading
import time
from concurrent import futures

import grpc
from google.protobuf import descriptor_pb2, descriptor_pool, message_factory

from . import binding as B

DEFAULT_REEF_ADDR = "localhost:34543"      # util/common.h:8
SERVICE = "reef.rpc.REEFService"

_T = descriptor_pb2.FieldDescriptorProto
_MESSAGES = {                               # reef.proto:25-79: name -> [(field, tag, type)]
    "LoadModelRequest": [("dir", 1, _T.TYPE_STRING), ("name", 2, _T.TYPE_STRING), ("qid", 3, _T.TYPE_INT32)],
    "LoadModelReply": [("succ", 1, _T.TYPE_BOOL), ("mid", 2, _T.TYPE_INT32)],
    "SetPriorityRequest": [("rt", 1, _T.TYPE_BOOL)],
    "SetPriorityReply": [("succ", 1, _T.TYPE_BOOL), ("qid", 2, _T.TYPE_INT32)],
    "RegisterBlobRequest": [("mid", 1, _T.TYPE_INT32), ("name", 2, _T.TYPE_STRING)],
    "RegisterBlobReply": [("succ", 1, _T.TYPE_BOOL), ("key", 2, _T.TYPE_STRING), ("size", 3, _T.TYPE_INT64)],
    "GetBlobRequest": [("key", 1, _T.TYPE_STRING)],
    "GetBlobReply": [("succ", 1, _T.TYPE_BOOL)],
    "SetBlobRequest": [("key", 1, _T.TYPE_STRING)],
    "SetBlobReply": [("succ", 1, _T.TYPE_BOOL)],
    "InferRequest": [("mid", 1, _T.TYPE_INT32), ("async", 2, _T.TYPE_BOOL)],
    "InferReply": [("succ", 1, _T.TYPE_BOOL), ("tid", 2, _T.TYPE_INT32)],
}
_METHODS = ["LoadModel", "SetPriority", "RegisterBlob", "GetBlob", "SetBlob", "Infer"]   # reef.proto:5-23


def _build_messages():
    fd = descriptor_pb2.FileDescriptorProto()
    fd.name = "reef.proto"
    fd.package = "reef.rpc"
    fd.syntax = "proto3"
    for mname, fields in _MESSAGES.items():
        m = fd.message_type.add()
        m.name = mname
        for fname, tag, ftype in fields:
            f = m.field.add()
            f.name, f.number, f.type, f.label = fname, tag, ftype, _T.LABEL_OPTIONAL
    svc = fd.service.add()
    svc.name = "REEFService"
    for meth in _METHODS:
        md = svc.method.add()
        md.name = meth
        md.input_type = ".reef.rpc.%sRequest" % meth
        md.output_type = ".reef.rpc.%sReply" % meth
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    return {n: message_factory.GetMessageClass(pool.FindMessageTypeByName("reef.rpc." + n)) for n in _MESSAGES}


MSG = _build_messages()


class SharedMemory:
    """POSIX shared memory as util/shared_memory.cpp:13-34 uses it: shm_open(key, O_CREAT|O_RDWR,
    0777), ftruncate, mmap; unlinked by its creator.  (shm_open of a name without a slash is the
    file of that name in /dev/shm.)"""

    def __init__(self, key, size, create=False):
        self.key, self.size, self.create = key, int(size), create
        path = os.path.join("/dev/shm", key)
        self.fd = os.open(path, (os.O_CREAT | os.O_RDWR) if create else os.O_RDWR, 0o777)
        os.ftruncate(self.fd, max(self.size, 1))
        self.map = mmap.mmap(self.fd, max(self.size, 1), mmap.MAP_SHARED, mmap.PROT_READ | mmap.PROT_WRITE)

    def address(self):
        return ctypes.addressof(ctypes.c_char.from_buffer(self.map))

    def array(self, dtype="float32"):
        import numpy as np
        return np.frombuffer(self.map, dtype=dtype, count=self.size // np.dtype(dtype).itemsize)

    def close(self):
        if self.map is not None:
            try:
                self.map.close()
            except BufferError:      # a view handed out by array() is still alive: the mapping goes with it
                pass
            self.map = None
            os.close(self.fd)
            if self.create:
                try:
                    os.unlink(os.path.join("/dev/shm", self.key))
                except FileNotFoundError:
                    pass


class REEFServer:
    """server/server.{h,cpp}: owns one scheduler (REEF mode, server.cpp:11) and the blobs."""

    def __init__(self, addr=DEFAULT_REEF_ADDR, mode=B.MODE_REEF, max_workers=16, measure_imported=True):
        self.addr = addr
        self.scheduler = B.Scheduler(mode)
        self.measure_imported = measure_imported   # profile an imported directory on the device (else: estimates)
        self.import_root = None                    # where directories of the reference are imported to
        self.import_mtx = threading.Lock()
        self.shms = {}                       # key -> (mid, name, SharedMemory)
        self.shm_mtx = threading.Lock()
        self.server = grpc.server(futures.ThreadPoolExecutor(max_workers=max_workers))
        handlers = {}
        for meth in _METHODS:
            handlers[meth] = grpc.unary_unary_rpc_method_handler(
                getattr(self, meth), request_deserializer=MSG[meth + "Request"].FromString,
                response_serializer=MSG[meth + "Reply"].SerializeToString)
        self.server.add_generic_rpc_handlers((grpc.method_handlers_generic_handler(SERVICE, handlers),))
        self.port = self.server.add_insecure_port(addr)
        if self.port == 0:
            raise RuntimeError("cannot listen on " + addr)

    # ---- life cycle (server.cpp:14-32) ----
    def run(self):
        self.server.start()
        self.scheduler.run()

    def wait(self):
        self.server.wait_for_termination()

    def shutdown(self):
        self.server.stop(0).wait()
        self.scheduler.shutdown()
        self.scheduler.close()
        with self.shm_mtx:
            for _, _, shm in self.shms.values():
                shm.close()
            self.shms.clear()
        if self.import_root is not None:
            shutil.rmtree(self.import_root, ignore_errors=True)
            self.import_root = None

    # ---- handlers ----
    def SetPriority(self, request, context):
        reply = MSG["SetPriorityReply"]()
        st, qid = self.scheduler.create_queue_status(B.QUEUE_RT if request.rt else B.QUEUE_BE)
        reply.succ = st == 0
        if st == 0:
            reply.qid = qid
        return reply

    def _model_dir(self, model_dir, name):
        """A directory written by the reference's own pipeline (generated kernel names, no `op`
        keys; scheduler.cpp:62-65 names its files) cannot be loaded as it is: its code objects are
        for another GPU.  Where a kernel table is packaged for it (reef_amd/legacy.py), it is
        imported once into a directory of this server and loaded from there, so a client of the
        reference can keep sending the paths it always sent."""
        from . import legacy
        try:
            with open(os.path.join(model_dir, name + ".json")) as f:
                kernels = json.load(f).get("kernels") or []
        except (OSError, ValueError):
            return model_dir
        if not kernels or "op" in kernels[0] or not os.path.exists(os.path.join(legacy.TABLE_DIR, name + ".json")):
            return model_dir
        with self.import_mtx:
            if self.import_root is None:
                self.import_root = tempfile.mkdtemp(prefix="reef_imported_")
            # one import per source: the directory it lies in and the state of its graph and
            # parameter files, so that another directory holding a model of the same name, or the
            # same directory after its files changed, is imported again instead of served stale
            ident = [os.path.realpath(model_dir)]
            for ext in (".json", ".param"):
                try:
                    st = os.stat(os.path.join(model_dir, name + ext))
                    ident.append("%s:%d:%d" % (ext, st.st_size, st.st_mtime_ns))
                except OSError:
                    ident.append(ext + ":absent")
            tag = hashlib.sha256("|".join(ident).encode()).hexdigest()[:16]
            out = os.path.join(self.import_root, tag, name)
            if not os.path.exists(os.path.join(out, name + ".json")):
                try:
                    legacy.import_model_dir(model_dir, name, out, measured_profile=self.measure_imported)
                except (legacy.ImportError_, OSError, RuntimeError):
                    return model_dir
        return out

    def LoadModel(self, request, context):
        reply = MSG["LoadModelReply"]()
        prefix = self._model_dir(request.dir, request.name) + "/" + request.name
        param = prefix + ".param"
        if not os.access(param, os.F_OK):
            param = ""
        mid = ctypes.c_uint32()
        st = B.lib().reef_scheduler_load_model_files(
            self.scheduler.h, (prefix + ".trans.co").encode(), (prefix + ".be.co").encode(),
            (prefix + ".json").encode(), (prefix + ".profile.json").encode(), param.encode(), ctypes.byref(mid))
        if st != 0:
            reply.succ = False
            return reply
        reply.mid = mid.value
        reply.succ = self.scheduler.bind_model_queue(request.qid, mid.value) == 0
        return reply

    def RegisterBlob(self, request, context):
        reply = MSG["RegisterBlobReply"]()
        reply.succ = False
        st, size = self.scheduler.get_data_size(request.mid, request.name)
        if st != 0:
            return reply
        key = "%d_%s" % (request.mid, request.name)
        reply.key, reply.size, reply.succ = key, size, True
        with self.shm_mtx:
            if key not in self.shms:
                self.shms[key] = (request.mid, request.name, SharedMemory(key, size, create=True))
        return reply

    def _blob(self, key):
        with self.shm_mtx:
            return self.shms.get(key)

    def GetBlob(self, request, context):
        reply = MSG["GetBlobReply"]()
        info = self._blob(request.key)
        if info is None:
            reply.succ = False
            return reply
        mid, _, shm = info
        st = B.lib().reef_scheduler_get_output(self.scheduler.h, mid, ctypes.c_void_p(shm.address()),
                                               ctypes.c_size_t(shm.size))
        reply.succ = st == 0
        return reply

    def SetBlob(self, request, context):
        reply = MSG["SetBlobReply"]()
        info = self._blob(request.key)
        if info is None:
            reply.succ = False
            return reply
        mid, name, shm = info
        st = B.lib().reef_scheduler_set_input(self.scheduler.h, mid, ctypes.c_void_p(shm.address()),
                                              ctypes.c_size_t(shm.size), name.encode())
        reply.succ = st == 0
        return reply

    def Infer(self, request, context):
        reply = MSG["InferReply"]()
        tid = ctypes.c_uint32()
        st = B.lib().reef_scheduler_new_task(self.scheduler.h, request.mid, ctypes.byref(tid))
        if st != 0:
            reply.succ = False
            return reply
        reply.succ = self.scheduler.wait_task(tid.value) == 0
        reply.tid = tid.value
        return reply


# ------------------------------------------------------------------------------------------
class ModelHandle:
    """client.cpp:57-141."""

    def __init__(self, calls, mid, model_dir, name):
        self._calls, self.mid, self.dir, self.name = calls, mid, model_dir, name
        self.input_blob = self.output_blob = None
        self.input_blob_key = self.output_blob_key = None

    def get_mid(self):
        return self.mid

    def infer(self):
        """Submits one inference and waits; returns (tid, latency in seconds)."""
        t0 = time.time()
        reply = self._calls["Infer"](MSG["InferRequest"](mid=self.mid))
        assert reply.succ, "Infer failed"
        return reply.tid, time.time() - t0

    def register_blob(self, name):
        reply = self._calls["RegisterBlob"](MSG["RegisterBlobRequest"](mid=self.mid, name=name))
        assert reply.succ, "RegisterBlob(%s) failed" % name
        return SharedMemory(reply.key, reply.size), reply.key

    def get_input_blob(self, name="data"):
        if self.input_blob is None:
            self.input_blob, self.input_blob_key = self.register_blob(name)
        return self.input_blob

    def get_output_blob(self, name="output"):
        if self.output_blob is None:
            self.output_blob, self.output_blob_key = self.register_blob(name)
        return self.output_blob

    def load_input(self):
        assert self.input_blob is not None
        assert self._calls["SetBlob"](MSG["SetBlobRequest"](key=self.input_blob_key)).succ, "SetBlob failed"

    def get_output(self):
        assert self.output_blob is not None
        assert self._calls["GetBlob"](MSG["GetBlobRequest"](key=self.output_blob_key)).succ, "GetBlob failed"

    def close(self):
        for b in (self.input_blob, self.output_blob):
            if b is not None:
                b.close()


class REEFClient:
    """client.cpp:11-55."""

    def __init__(self, addr=DEFAULT_REEF_ADDR):
        self.channel = grpc.insecure_channel(addr)
        self.calls = {
            meth: self.channel.unary_unary("/%s/%s" % (SERVICE, meth),
                                           request_serializer=MSG[meth + "Request"].SerializeToString,
                                           response_deserializer=MSG[meth + "Reply"].FromString)
            for meth in _METHODS}
        self.qid = None
        self.models = []

    def init(self, real_time):
        reply = self.calls["SetPriority"](MSG["SetPriorityRequest"](rt=bool(real_time)))
        assert reply.succ, "SetPriority failed"
        self.qid = reply.qid
        return True

    def load_model(self, model_dir, name):
        reply = self.calls["LoadModel"](MSG["LoadModelRequest"](dir=model_dir, name=name, qid=self.qid))
        assert reply.succ, "LoadModel(%s/%s) failed" % (model_dir, name)
        m = ModelHandle(self.calls, reply.mid, model_dir, name)
        self.models.append(m)
        return m

    def close(self):
        for m in self.models:
            m.close()
        self.channel.close()


def main(argv):
    usage = ("usage: python -m reef_amd.rpc server [addr]\n"
             "       python -m reef_amd.rpc client model_dir model_name real_time\n"
             "       python -m reef_amd.rpc client_cont model_dir model_name real_time sleep_time(ms)")
    if len(argv) < 2:
        print(usage, file=sys.stderr)
        return 1
    if argv[1] == "server":                       # src/example/rpc_server.cpp
        server = REEFServer(argv[2] if len(argv) > 2 else DEFAULT_REEF_ADDR)
        server.run()
        server.wait()
        return 0
    if argv[1] in ("client", "client_cont") and len(argv) >= 5:   # src/example/rpc_client{,_cont}.cpp
        client = REEFClient(DEFAULT_REEF_ADDR)
        client.init(int(argv[4]))
        print("loading '%s' from '%s'" % (argv[3], argv[2]))
        model = client.load_model(argv[2], argv[3])
        print("submit inference requests")
        sleep_ms = int(argv[5]) if argv[1] == "client_cont" and len(argv) > 5 else None
        while True:
            _, lat = model.infer()
            print("client %d inference latency: %.3f ms" % (model.get_mid(), lat * 1e3), flush=True)
            if sleep_ms is None:
                break
            time.sleep(sleep_ms / 1e3)
        client.close()
        return 0
    print(usage, file=sys.stderr)
    return 1


if __name__ == "__main__":
    sys.exit(main(sys.argv))
