import ctypes
import sys
import os

_HERE = os.path.dirname(os.path.abspath(__file__))

F16, F32, F64, C64 = 0, 1, 2, 3
DTYPE_SIZE = {F16: 2, F32: 4, F64: 8, C64: 8}

OK, UNSUPPORTED = 0, 1
ERR_INVALID, ERR_NOT_BUILT, ERR_WORKSPACE, ERR_INPUTS, ERR_DEVICE = -1, -2, -3, -4, -5

EXPORTS = [
    "es_km_create",
    "es_km_destroy",
    "es_km_last_error",
    "es_km_build",
    "es_km_workspace_size",
    "es_km_execute",
    "es_km_execute_static_workspace",
    "es_km_describe",
    "es_km_touch",
    "es_km_touch_batch",
    "es_km_fill_constant",
    "es_km_fill_lowertri",
    "es_km_codegen_source",
    "es_km_scalarop_roundtrip",
    "es_km_scalarop_simplify",
    "es_km_merge_adjacent_dims",
    "es_km_probe_mfma_f16",
    "es_km_graph_create",
    "es_km_graph_destroy",
    "es_km_graph_add_einsummable",
    "es_km_graph_add_touch",
    "es_km_graph_add_fill_constant",
    "es_km_graph_add_fill_lowertri",
    "es_km_graph_add_copy",
    "es_km_graph_add_memory_dependencies",
    "es_km_graph_optimize",
    "es_km_graph_node_describe",
    "es_km_graph_node_source",
    "es_km_graph_finalize",
    "es_km_graph_run",
    "es_km_graph_node_info",
    "es_km_graph_cross_stream_waits",
    "es_km_graph_launches",
    "es_km_graph_launch_node",
    "es_km_graph_node_workspace",
    "es_km_graph_node_group",
    "es_km_workspace_pool_create",
    "es_km_workspace_pool_destroy",
    "es_km_workspace_pool_acquire",
    "es_km_workspace_pool_release",
    "es_km_workspace_pool_blocks",
    "es_km_stream_pool_create",
    "es_km_stream_pool_destroy",
    "es_km_stream_pool_try_acquire",
    "es_km_stream_pool_release",
    "es_km_graph_add_dummy",
    "es_km_graph_add_placeholder",
    "es_km_graph_add_evict",
    "es_km_graph_add_load",
    "es_km_graph_declare_storage",
    "es_km_graph_storage_write",
    "es_km_graph_storage_read",
    "es_km_graph_load_memgraph",
    "es_km_graph_num_nodes",
    "es_km_graph_arena_bytes",
    "es_km_graph_node_mems",
    "es_km_memgraph_describe",
]


class KmError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("es_km error %d: %s" % (code, message))
        self.code = code


def lib_path():
    return os.path.join(_HERE, "libes_km.so")


_lib = None


def load_library():
    """Load libes_km.so.  There is no fallback: a missing library is an error."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise ImportError(
            "%s is missing: build it with `python -m einsummable_amd.build`" % path
        )
    # One HIP runtime per process.  PyTorch wheels bundle their own libamdhip64 / libhiprtc
    # under the same sonames as /opt/rocm's: loaded first, they also satisfy this library's
    # NEEDED entries; loaded second, they come in as a second runtime beside /opt/rocm's, and
    # the second one to touch the device finds none.  The tests and bench.py take device
    # memory and streams from torch, so torch goes first whenever it is installed.  (A C++
    # host that links this library has no torch in it and uses /opt/rocm's runtime.)
    if "torch" not in sys.modules:
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
    lib = ctypes.CDLL(path)
    lib.es_km_create.restype = ctypes.c_void_p
    lib.es_km_create.argtypes = [ctypes.c_int]
    lib.es_km_destroy.argtypes = [ctypes.c_void_p]
    lib.es_km_last_error.restype = ctypes.c_char_p
    lib.es_km_last_error.argtypes = [ctypes.c_void_p]
    desc = [
        ctypes.c_void_p,  # join_shape
        ctypes.c_int,
        ctypes.c_void_p,  # inns_flat
        ctypes.c_void_p,  # inns_offsets
        ctypes.c_int,
        ctypes.c_int,
        ctypes.c_char_p,
        ctypes.c_char,
    ]
    lib.es_km_build.argtypes = [ctypes.c_void_p] + desc + [ctypes.c_void_p]
    lib.es_km_workspace_size.argtypes = [ctypes.c_void_p] + desc + [ctypes.c_void_p]
    lib.es_km_execute.argtypes = [ctypes.c_void_p] + desc + [
        ctypes.c_void_p,
        ctypes.c_void_p,
        ctypes.c_void_p,
        ctypes.c_int,
        ctypes.c_void_p,
        ctypes.c_uint64,
    ]
    lib.es_km_execute_static_workspace.argtypes = [ctypes.c_void_p] + desc + [
        ctypes.c_void_p,
        ctypes.c_void_p,
        ctypes.c_void_p,
        ctypes.c_int,
    ]
    lib.es_km_describe.argtypes = [ctypes.c_void_p] + desc + [ctypes.c_void_p, ctypes.c_size_t]
    lib.es_km_touch.argtypes = [
        ctypes.c_void_p,
        ctypes.c_void_p,
        ctypes.c_int,
        ctypes.c_char,
        ctypes.c_int,
        ctypes.c_void_p,
        ctypes.c_void_p,
        ctypes.c_void_p,
    ]
    lib.es_km_touch_batch.argtypes = [
        ctypes.c_void_p,
        ctypes.c_int,
        ctypes.c_void_p,
        ctypes.c_void_p,
        ctypes.c_char_p,
        ctypes.c_int,
        ctypes.c_void_p,
        ctypes.c_void_p,
        ctypes.c_void_p,
    ]
    lib.es_km_fill_constant.argtypes = [
        ctypes.c_void_p,
        ctypes.c_int,
        ctypes.c_uint64,
        ctypes.c_uint64,
        ctypes.c_void_p,
        ctypes.c_void_p,
    ]
    lib.es_km_fill_lowertri.argtypes = [
        ctypes.c_void_p,
        ctypes.c_int,
        ctypes.c_uint64,
        ctypes.c_uint64,
        ctypes.c_uint64,
        ctypes.c_uint64,
        ctypes.c_int64,
        ctypes.c_void_p,
        ctypes.c_void_p,
    ]
    lib.es_km_probe_mfma_f16.restype = ctypes.c_double
    lib.es_km_probe_mfma_f16.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                         ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.es_km_codegen_source.argtypes = desc + [ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t]
    lib.es_km_scalarop_roundtrip.argtypes = [ctypes.c_char_p, ctypes.c_void_p, ctypes.c_size_t,
                                             ctypes.c_void_p, ctypes.c_void_p]
    lib.es_km_merge_adjacent_dims.argtypes = desc + [ctypes.c_void_p, ctypes.c_void_p,
                                                     ctypes.c_void_p, ctypes.c_void_p,
                                                     ctypes.c_void_p, ctypes.c_size_t]
    V, I, U64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_uint64
    lib.es_km_graph_create.restype = V
    lib.es_km_graph_create.argtypes = [V]
    lib.es_km_graph_destroy.argtypes = [V]
    lib.es_km_graph_add_einsummable.argtypes = [V] + desc + [V, V, I, V, I]
    lib.es_km_graph_add_touch.argtypes = [V, V, I, ctypes.c_char, I, I, V, V, V, I]
    lib.es_km_graph_add_fill_constant.argtypes = [V, I, U64, U64, U64, U64, V, I]
    lib.es_km_graph_add_fill_lowertri.argtypes = [V, I, U64, U64, U64, U64, ctypes.c_int64, U64,
                                                  U64, V, I]
    lib.es_km_graph_add_copy.argtypes = [V, U64, U64, U64, V, I]
    lib.es_km_graph_add_memory_dependencies.argtypes = [V]
    lib.es_km_graph_optimize.argtypes = [V, ctypes.POINTER(ctypes.c_int)]
    lib.es_km_graph_node_describe.restype = ctypes.c_int64
    lib.es_km_graph_node_describe.argtypes = [V, I, ctypes.c_char_p, U64]
    lib.es_km_graph_node_source.restype = ctypes.c_int64
    lib.es_km_graph_node_source.argtypes = [V, I, I, ctypes.c_char_p, U64]
    lib.es_km_graph_finalize.argtypes = [V, I]
    lib.es_km_graph_run.argtypes = [V, V, V]
    lib.es_km_graph_node_info.argtypes = [V, I, V, V, V, I, V]
    lib.es_km_graph_cross_stream_waits.argtypes = [V]
    lib.es_km_graph_launches.argtypes = [V]
    lib.es_km_graph_launch_node.argtypes = [V, I, V, V, V, U64, I, V, V]
    lib.es_km_graph_node_workspace.argtypes = [V, I, V]
    lib.es_km_graph_node_group.argtypes = [V, I]
    lib.es_km_workspace_pool_create.restype = V
    lib.es_km_workspace_pool_create.argtypes = [I]
    lib.es_km_workspace_pool_destroy.argtypes = [V]
    lib.es_km_workspace_pool_acquire.restype = V
    lib.es_km_workspace_pool_acquire.argtypes = [V, U64, V]
    lib.es_km_workspace_pool_release.argtypes = [V, V]
    lib.es_km_workspace_pool_blocks.argtypes = [V]
    lib.es_km_stream_pool_create.restype = V
    lib.es_km_stream_pool_create.argtypes = [I, I]
    lib.es_km_stream_pool_destroy.argtypes = [V]
    lib.es_km_stream_pool_try_acquire.restype = V
    lib.es_km_stream_pool_try_acquire.argtypes = [V]
    lib.es_km_stream_pool_release.argtypes = [V, V]
    lib.es_km_graph_add_dummy.argtypes = [V, U64, U64, V, I]
    lib.es_km_graph_add_placeholder.argtypes = [V, U64, U64, V, I]
    lib.es_km_graph_add_evict.argtypes = [V, U64, U64, I, V, I]
    lib.es_km_graph_add_load.argtypes = [V, I, U64, U64, V, I]
    lib.es_km_graph_declare_storage.argtypes = [V, I, U64]
    lib.es_km_graph_storage_write.argtypes = [V, I, V, U64]
    lib.es_km_graph_storage_read.argtypes = [V, I, V, U64]
    lib.es_km_graph_load_memgraph.argtypes = [V, V, U64, I, V, V, I]
    lib.es_km_graph_num_nodes.argtypes = [V]
    lib.es_km_graph_arena_bytes.argtypes = [V]
    lib.es_km_graph_arena_bytes.restype = U64
    lib.es_km_graph_node_mems.argtypes = [V, I, V, V, V, I, V]
    lib.es_km_memgraph_describe.argtypes = [V, U64, V, U64]
    lib.es_km_memgraph_describe.restype = ctypes.c_int64
    _lib = lib
    return lib


def _castable_char(c):
    return (c.encode() if c else b"\0")


class Einsummable:
    """The fields of einsummable_t (src/einsummable/einsummable.h:8-20); `join` is the
    scalarop text, `castable` one of '+', 'x', 'v', '^' or None."""

    def __init__(self, join_shape, inns, out_rank, join, castable=None):
        self.join_shape = [int(x) for x in join_shape]
        self.inns = [list(map(int, inn)) for inn in inns]
        self.out_rank = int(out_rank)
        # aggregated modes are numbered in order of first appearance, as the reference's
        # constructor does (src/einsummable/einsummable.cc:32-93): join_shape is indexed by
        # the numbers after this step, so inn_shape() must see them too
        renamed = {}
        for inn in self.inns:
            for i, m in enumerate(inn):
                if m >= self.out_rank:
                    inn[i] = renamed.setdefault(m, self.out_rank + len(renamed))
        self.join = join
        self.castable = castable
        flat, offs = [], [0]
        for inn in self.inns:
            flat.extend(inn)
            offs.append(len(flat))
        self._shape = (ctypes.c_uint64 * len(self.join_shape))(*self.join_shape)
        self._flat = (ctypes.c_int * max(len(flat), 1))(*flat)
        self._offs = (ctypes.c_int * len(offs))(*offs)
        self._join = join.encode()
        self._args = (
            ctypes.cast(self._shape, ctypes.c_void_p),
            len(self.join_shape),
            ctypes.cast(self._flat, ctypes.c_void_p),
            ctypes.cast(self._offs, ctypes.c_void_p),
            len(self.inns),
            self.out_rank,
            self._join,
            _castable_char(castable),
        )

    @staticmethod
    def from_str(s, sizes, join, castable=None):
        """'ij,jk->ik' with sizes {'i': .., 'j': .., 'k': ..} (parse_str,
        src/einsummable/einsummable.cc:364-441)."""
        lhs, out = s.split("->")
        ids = {}
        for ch in out:
            ids[ch] = len(ids)
        inns = []
        for word in lhs.split(","):
            inn = []
            for ch in word:
                if ch not in ids:
                    ids[ch] = len(ids)
                inn.append(ids[ch])
            inns.append(inn)
        shape = [0] * len(ids)
        for ch, i in ids.items():
            shape[i] = sizes[ch]
        return Einsummable(shape, inns, len(out), join, castable)

    def out_nelem(self):
        n = 1
        for d in self.join_shape[: self.out_rank]:
            n *= d
        return n

    def inn_shape(self, k):
        return [self.join_shape[m] for m in self.inns[k]]


class Touch:
    """touch_t (src/einsummable/touch.h:25-29): selection of
    (d_inn, d_out, offset_inn, offset_out, size), optional castable, dtype."""

    def __init__(self, selection, castable, dtype):
        self.selection = [tuple(int(v) for v in d) for d in selection]
        self.castable = castable
        self.dtype = dtype
        flat = [v for d in self.selection for v in d]
        self._dims = (ctypes.c_uint64 * len(flat))(*flat)


class TouchBatch:
    """Flattened descriptors of a list of Touch objects (built once, reused per call)."""

    def __init__(self, touches):
        flat = [v for t in touches for d in t.selection for v in d]
        self.n = len(touches)
        self.dtype = touches[0].dtype if touches else F32
        self.dims = (ctypes.c_uint64 * max(len(flat), 1))(*flat)
        self.ranks = (ctypes.c_int * max(self.n, 1))(*[len(t.selection) for t in touches])
        self.castables = b"".join(_castable_char(t.castable) for t in touches) + b"\0"


def codegen_source(e, compile=False):
    lib = load_library()
    buf = ctypes.create_string_buffer(1 << 16)
    rc = lib.es_km_codegen_source(*e._args, int(compile), ctypes.cast(buf, ctypes.c_void_p),
                                  1 << 16)
    if rc != OK:
        raise KmError(rc, lib.es_km_last_error(None).decode("utf-8", "replace"))
    return buf.value.decode("utf-8", "replace")


def scalarop_roundtrip(text):
    """(printed text, out dtype, number of holes) from the library's own scalarop parser."""
    lib = load_library()
    buf = ctypes.create_string_buffer(8192)
    od, n = ctypes.c_int(), ctypes.c_int()
    rc = lib.es_km_scalarop_roundtrip(text.encode(), ctypes.cast(buf, ctypes.c_void_p), 8192,
                                      ctypes.byref(od), ctypes.byref(n))
    if rc != OK:
        raise KmError(rc, lib.es_km_last_error(None).decode("utf-8", "replace"))
    return buf.value.decode("utf-8", "replace"), od.value, n.value


def scalarop_simplify(text, variables=None):
    """The reference's canonical form of a scalarop text, after replacing the named variables
    (a dict name -> value) by constants."""
    lib = load_library()
    items = sorted((variables or {}).items())
    names = (ctypes.c_char_p * max(len(items), 1))(*[k.encode() for k, _ in items])
    vals = (ctypes.c_double * max(len(items), 1))(*[float(v) for _, v in items])
    buf = ctypes.create_string_buffer(1 << 14)
    lib.es_km_scalarop_simplify.argtypes = [ctypes.c_char_p, ctypes.c_void_p, ctypes.c_void_p,
                                            ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t]
    rc = lib.es_km_scalarop_simplify(text.encode(), names, vals, len(items), buf, len(buf))
    if rc != OK:
        raise KmError(rc, lib.es_km_last_error(None).decode("utf-8", "replace"))
    return buf.value.decode()


def merge_adjacent_dims(e):
    """(join_shape, inns, out_rank, str) of e.merge_adjacent_dims() from the library."""
    lib = load_library()
    n_modes = sum(len(i) for i in e.inns)
    js = (ctypes.c_uint64 * len(e.join_shape))()
    flat = (ctypes.c_int * max(n_modes, 1))()
    offs = (ctypes.c_int * (len(e.inns) + 1))()
    orank = ctypes.c_int()
    buf = ctypes.create_string_buffer(256)
    rc = lib.es_km_merge_adjacent_dims(*e._args, js, flat, offs, ctypes.byref(orank), buf, 256)
    if rc < 0:
        raise KmError(rc, lib.es_km_last_error(None).decode("utf-8", "replace"))
    inns = [[flat[i] for i in range(offs[k], offs[k + 1])] for k in range(len(e.inns))]
    return [int(js[i]) for i in range(rc)], inns, orank.value, buf.value.decode("utf-8", "replace")


class KernelManager:
    """kernel_manager_t(device): build / workspace_size / __call__ / touch / fills on raw
    device addresses (ints) and a raw hipStream_t (int, 0 = default stream)."""

    def __init__(self, device=0):
        self._lib = load_library()
        # A process that also uses torch for device memory must let torch set the device up
        # before the library's first HIP call (the other way round torch finds no GPU).
        torch = sys.modules.get("torch")
        if torch is not None and torch.cuda.is_available():
            torch.cuda.init()
        self._h = self._lib.es_km_create(int(device))
        if not self._h:
            raise KmError(ERR_DEVICE, self._lib.es_km_last_error(None).decode("utf-8", "replace"))

    def close(self):
        if self._h:
            self._lib.es_km_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _fail(self, rc):
        raise KmError(rc, self._lib.es_km_last_error(self._h).decode("utf-8", "replace"))

    def build(self, e):
        """Workspace bytes, or None when unsupported (the reference returns nullopt)."""
        ws = ctypes.c_uint64(0)
        rc = self._lib.es_km_build(self._h, *e._args, ctypes.byref(ws))
        if rc == UNSUPPORTED:
            return None
        if rc != OK:
            self._fail(rc)
        return ws.value

    def workspace_size(self, e):
        ws = ctypes.c_uint64(0)
        rc = self._lib.es_km_workspace_size(self._h, *e._args, ctypes.byref(ws))
        if rc != OK:
            self._fail(rc)
        return ws.value

    def describe(self, e):
        buf = ctypes.create_string_buffer(256)
        rc = self._lib.es_km_describe(self._h, *e._args, ctypes.cast(buf, ctypes.c_void_p), 256)
        if rc != OK:
            self._fail(rc)
        return buf.value.decode("utf-8", "replace")

    def __call__(self, e, stream, out, inns, workspace=None):
        ptrs = (ctypes.c_void_p * max(len(inns), 1))(*inns)
        ws_ptr, ws_size = workspace if workspace else (None, 0)
        rc = self._lib.es_km_execute(self._h, *e._args, stream, out, ptrs, len(inns), ws_ptr,
                                     ws_size)
        if rc != OK:
            self._fail(rc)

    def execute_static_workspace(self, e, stream, out, inns):
        """Like __call__, with the library's own 64 MiB workspace: allocates nothing."""
        ptrs = (ctypes.c_void_p * max(len(inns), 1))(*inns)
        rc = self._lib.es_km_execute_static_workspace(self._h, *e._args, stream, out, ptrs,
                                                      len(inns))
        if rc != OK:
            self._fail(rc)

    def touch(self, t, stream, out, inn):
        rc = self._lib.es_km_touch(self._h, ctypes.cast(t._dims, ctypes.c_void_p),
                                   len(t.selection), _castable_char(t.castable), t.dtype, stream,
                                   out, inn)
        if rc != OK:
            self._fail(rc)

    def touch_batch(self, touches, stream, out, inns):
        """Apply `touches` (all into `out`) in list order with one launch per 32 touches."""
        batch = TouchBatch(touches) if not isinstance(touches, TouchBatch) else touches
        ptrs = (ctypes.c_void_p * max(len(inns), 1))(*inns)
        rc = self._lib.es_km_touch_batch(self._h, batch.n, ctypes.cast(batch.dims, ctypes.c_void_p),
                                         ctypes.cast(batch.ranks, ctypes.c_void_p),
                                         batch.castables, batch.dtype, stream, out, ptrs)
        if rc != OK:
            self._fail(rc)

    def probe_mfma_f16(self, operands, scratch, blocks, iters, stream):
        return self._lib.es_km_probe_mfma_f16(self._h, operands, scratch, blocks, iters, stream)

    def constant_fill(self, dtype, value_bits, nelem, stream, out):
        rc = self._lib.es_km_fill_constant(self._h, dtype, value_bits, nelem, stream, out)
        if rc != OK:
            self._fail(rc)

    def lowerTri_fill(self, dtype, lower_bits, upper_bits, nrow, ncol, start, stream, out):
        rc = self._lib.es_km_fill_lowertri(self._h, dtype, lower_bits, upper_bits, nrow, ncol,
                                           start, stream, out)
        if rc != OK:
            self._fail(rc)


NodeCallback = ctypes.CFUNCTYPE(None, ctypes.c_void_p)


class WorkspacePool:
    """gpu_workspace_manager_t (src/engine/gpu/workspace.cc:48-91) over the C ABI."""

    def __init__(self, device=0):
        self._lib = load_library()
        self._p = self._lib.es_km_workspace_pool_create(int(device))
        if not self._p:
            raise KmError(ERR_DEVICE, self._lib.es_km_last_error(None).decode("utf-8", "replace"))

    def acquire(self, nbytes):
        got = ctypes.c_uint64(0)
        ptr = self._lib.es_km_workspace_pool_acquire(self._p, int(nbytes), ctypes.byref(got))
        if not ptr:
            raise KmError(ERR_DEVICE, self._lib.es_km_last_error(None).decode("utf-8", "replace"))
        return ptr, got.value

    def release(self, ptr):
        rc = self._lib.es_km_workspace_pool_release(self._p, ptr)
        if rc != OK:
            raise KmError(rc, self._lib.es_km_last_error(None).decode("utf-8", "replace"))

    def blocks(self):
        return self._lib.es_km_workspace_pool_blocks(self._p)

    def close(self):
        if self._p:
            self._lib.es_km_workspace_pool_destroy(self._p)
            self._p = None


class StreamPool:
    """streampool_manager_t (src/engine/gpu/stream_pool.cc:42-75) over the C ABI."""

    def __init__(self, device=0, n_streams=4):
        self._lib = load_library()
        self._p = self._lib.es_km_stream_pool_create(int(device), int(n_streams))
        if not self._p:
            raise KmError(ERR_DEVICE, self._lib.es_km_last_error(None).decode("utf-8", "replace"))

    def try_acquire(self):
        return self._lib.es_km_stream_pool_try_acquire(self._p)

    def release(self, stream):
        rc = self._lib.es_km_stream_pool_release(self._p, stream)
        if rc != OK:
            raise KmError(rc, self._lib.es_km_last_error(None).decode("utf-8", "replace"))

    def close(self):
        if self._p:
            self._lib.es_km_stream_pool_destroy(self._p)
            self._p = None


class ApplyGraph:
    """The exec-node layer (include/es_km.h, es_km_graph_*): apply / fill / copy nodes over
    one device arena with dependencies, placed on a pool of streams at finalize() and
    enqueued by run() without any host synchronisation.  `km=None` gives a graph that can be
    planned and inspected without a device."""

    def __init__(self, km=None):
        self._lib = load_library()
        self._km = km
        self._g = self._lib.es_km_graph_create(km._h if km is not None else None)
        if not self._g:
            raise KmError(ERR_DEVICE, "es_km_graph_create failed")

    def close(self):
        if self._g:
            self._lib.es_km_graph_destroy(self._g)
            self._g = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, rc):
        if rc < 0:
            h = self._km._h if self._km is not None else None
            raise KmError(rc, self._lib.es_km_last_error(h).decode("utf-8", "replace"))
        return rc

    @staticmethod
    def _mems(mems):
        offs = (ctypes.c_uint64 * len(mems))(*[int(m[0]) for m in mems])
        sizes = (ctypes.c_uint64 * len(mems))(*[int(m[1]) for m in mems])
        return offs, sizes

    @staticmethod
    def _deps(deps):
        deps = list(deps or [])
        return (ctypes.c_int * max(len(deps), 1))(*deps), len(deps)

    def add_einsummable(self, e, mems, deps=None):
        """mems: [(offset, size)] with the output first, then the inputs."""
        offs, sizes = self._mems(mems)
        d, nd = self._deps(deps)
        return self._check(self._lib.es_km_graph_add_einsummable(
            self._g, *e._args, offs, sizes, len(mems), d, nd))

    def add_touch(self, t, group, mems, deps=None):
        offs, sizes = self._mems(mems)
        d, nd = self._deps(deps)
        return self._check(self._lib.es_km_graph_add_touch(
            self._g, ctypes.cast(t._dims, ctypes.c_void_p), len(t.selection),
            _castable_char(t.castable), t.dtype, int(group), offs, sizes, d, nd))

    def add_constant_fill(self, dtype, value_bits, nelem, mem, deps=None):
        d, nd = self._deps(deps)
        return self._check(self._lib.es_km_graph_add_fill_constant(
            self._g, dtype, value_bits, nelem, int(mem[0]), int(mem[1]), d, nd))

    def add_lowertri_fill(self, dtype, lower_bits, upper_bits, nrow, ncol, start, mem, deps=None):
        d, nd = self._deps(deps)
        return self._check(self._lib.es_km_graph_add_fill_lowertri(
            self._g, dtype, lower_bits, upper_bits, nrow, ncol, start, int(mem[0]), int(mem[1]),
            d, nd))

    def add_copy(self, dst_offset, src_offset, size, deps=None):
        d, nd = self._deps(deps)
        return self._check(self._lib.es_km_graph_add_copy(self._g, dst_offset, src_offset, size,
                                                          d, nd))

    def add_memory_dependencies(self):
        self._check(self._lib.es_km_graph_add_memory_dependencies(self._g))

    def optimize(self):
        """Absorbs whole-range copies and single-reader elementwise producers into their
        neighbours (es_km_graph_optimize); returns how many nodes were absorbed."""
        n = ctypes.c_int(0)
        self._check(self._lib.es_km_graph_optimize(self._g, ctypes.byref(n)))
        return n.value

    def finalize(self, n_streams=1):
        self._check(self._lib.es_km_graph_finalize(self._g, int(n_streams)))

    def run(self, stream, arena):
        self._check(self._lib.es_km_graph_run(self._g, stream, arena))

    def node_info(self, node):
        """(launch position, stream index, [dependencies]) after finalize."""
        pos, st, n = ctypes.c_int(-1), ctypes.c_int(-1), ctypes.c_int(0)
        deps = (ctypes.c_int * 4096)()
        self._check(self._lib.es_km_graph_node_info(self._g, node, ctypes.byref(pos),
                                                    ctypes.byref(st), deps, 4096, ctypes.byref(n)))
        return pos.value, st.value, list(deps[:min(n.value, 4096)])

    def describe(self, node):
        """"<kind> <offset>:<size> ... | <einsummable key>" of a node."""
        buf = ctypes.create_string_buffer(1 << 14)
        n = self._lib.es_km_graph_node_describe(self._g, int(node), buf, len(buf))
        if n < 0:
            raise KmError(int(n), "no such node")
        return buf.value.decode()

    def node_source(self, node, compile=False):
        """HIP source of the generated kernel of a node ("" when it has none); `compile`
        also compiles it for gfx950, which needs no device."""
        buf = ctypes.create_string_buffer(1 << 17)
        n = self._lib.es_km_graph_node_source(self._g, int(node), int(compile), buf, len(buf))
        self._check(n)
        return buf.value.decode()

    def cross_stream_waits(self):
        return self._check(self._lib.es_km_graph_cross_stream_waits(self._g))

    def launches(self):
        return self._check(self._lib.es_km_graph_launches(self._g))

    def node_workspace(self, i):
        ws = ctypes.c_uint64(0)
        self._check(self._lib.es_km_graph_node_workspace(self._g, int(i), ctypes.byref(ws)))
        return ws.value

    def node_group(self, i):
        return self._lib.es_km_graph_node_group(self._g, int(i))

    def launch_node(self, i, stream, arena, workspace=None, first_in_group=-1, callback=None,
                    user=None):
        """Enqueue one node on `stream`; `callback` is a NodeCallback (keep it alive until it
        has run) called with `user` (an int) when the node's work is done."""
        ws_ptr, ws_size = workspace if workspace else (None, 0)
        self._check(self._lib.es_km_graph_launch_node(
            self._g, int(i), stream, arena, ws_ptr, ws_size, int(first_in_group),
            ctypes.cast(callback, ctypes.c_void_p) if callback is not None else None, user))

    def add_dummy(self, mem=(0, 0), deps=None, is_del=True):
        """A node that launches nothing.  With a range it stands for the range's del, unless
        is_del is False (a placeholder: the range of an input or an alloc)."""
        d, nd = self._deps(deps)
        f = self._lib.es_km_graph_add_dummy if is_del else self._lib.es_km_graph_add_placeholder
        return self._check(f(self._g, int(mem[0]), int(mem[1]), d, nd))

    def add_evict(self, mem, storage_id, deps=None):
        d, nd = self._deps(deps)
        return self._check(self._lib.es_km_graph_add_evict(self._g, int(mem[0]), int(mem[1]),
                                                           int(storage_id), d, nd))

    def add_load(self, storage_id, mem, deps=None):
        d, nd = self._deps(deps)
        return self._check(self._lib.es_km_graph_add_load(self._g, int(storage_id), int(mem[0]),
                                                          int(mem[1]), d, nd))

    def declare_storage(self, storage_id, size):
        self._check(self._lib.es_km_graph_declare_storage(self._g, int(storage_id), int(size)))

    def storage_write(self, storage_id, data):
        """data: bytes-like, copied into the slot (after finalize)."""
        data = bytes(data)
        self._check(self._lib.es_km_graph_storage_write(self._g, int(storage_id), data,
                                                        len(data)))

    def storage_read(self, storage_id, size):
        buf = ctypes.create_string_buffer(int(size))
        self._check(self._lib.es_km_graph_storage_read(self._g, int(storage_id), buf, int(size)))
        return buf.raw

    def load_memgraph(self, wire, loc=0, scalar_vars=None):
        """Append every node of a serialized MemGraph (the reference's memgraph_t::to_wire
        bytes) for compute location `loc`; node ids equal the memgraph's."""
        wire = bytes(wire)
        items = sorted((scalar_vars or {}).items())
        names = (ctypes.c_char_p * max(len(items), 1))(*[k.encode() for k, _ in items])
        vals = (ctypes.c_double * max(len(items), 1))(*[float(v) for _, v in items])
        return self._check(self._lib.es_km_graph_load_memgraph(
            self._g, wire, len(wire), int(loc), names, vals, len(items)))

    def num_nodes(self):
        return self._check(self._lib.es_km_graph_num_nodes(self._g))

    def arena_bytes(self):
        return int(self._lib.es_km_graph_arena_bytes(self._g))

    NODE_KINDS = ("einsummable", "touch", "constant", "lowertri", "copy", "dummy", "evict",
                  "load", "chain")

    def node_mems(self, node):
        """(kind name, [(offset, size)]) of a node."""
        kind, n = ctypes.c_int(-1), ctypes.c_int(0)
        offs, sizes = (ctypes.c_uint64 * 64)(), (ctypes.c_uint64 * 64)()
        self._check(self._lib.es_km_graph_node_mems(self._g, node, ctypes.byref(kind), offs,
                                                    sizes, 64, ctypes.byref(n)))
        k = min(n.value, 64)
        return self.NODE_KINDS[kind.value], [(offs[i], sizes[i]) for i in range(k)]


def memgraph_describe(wire):
    """One line per node of a serialized MemGraph, every decoded field in a fixed order."""
    lib = load_library()
    wire = bytes(wire)
    n = lib.es_km_memgraph_describe(wire, len(wire), None, 0)
    if n < 0:
        raise KmError(int(n), lib.es_km_last_error(None).decode("utf-8", "replace"))
    buf = ctypes.create_string_buffer(int(n) + 1)
    lib.es_km_memgraph_describe(wire, len(wire), buf, int(n) + 1)
    return buf.value.decode("utf-8", "replace")
