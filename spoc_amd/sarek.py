"""`Vector`, `Transfer` and `Execute` by the reference's names (sarek/core/Vector.ml,
sarek/core/Transfer.ml, sarek/sarek/Execute.ml), over the native host layer of libsarek_hip:
a program written against them reads like the OCaml it mirrors,

    a = Vector.create(Vector.float32, n)
    for i in range(n): a[i] = ...                      # Vector.set
    Execute.run_vectors(ir=kernel_ir, args=[Execute.Vec(a), Execute.Int(n)],
                        block=Execute.dims1d(256), grid=Execute.dims1d((n + 255) // 256))
    Transfer.flush()
    result = a.to_array()                              # downloads: the launch left `a` Stale_CPU

Location states, what moves when, and the error texts are the native layer's, which follows
the reference state by state.
"""
import ctypes as C

import numpy as np

from . import hip

CPU, GPU, Both, Stale_CPU, Stale_GPU = "CPU", "GPU", "Both", "Stale_CPU", "Stale_GPU"
_LOCATIONS = (CPU, GPU, Both, Stale_CPU, Stale_GPU)


class Device:
    """sarek/core/Device.ml for the one framework of this library: enumeration, the capabilities
    record (spoc/framework/Framework_sig.ml:26-41, filled as sarek-cuda/Cuda_plugin_base.ml:177-195
    fills it) and the queries over it."""
    framework = "HIP"

    def __init__(self, dev_id, info):
        self.id = self.backend_id = dev_id
        self.name = info.name.decode()
        self.arch = info.gcn_arch.decode()
        self.capabilities = dict(
            max_threads_per_block=info.max_threads_per_block, max_block_dims=tuple(info.max_block_dim),
            max_grid_dims=tuple(info.max_grid_dim), shared_mem_per_block=info.shared_mem_per_block,
            total_global_mem=info.total_global_mem, compute_capability=(info.compute_major, info.compute_minor),
            supports_fp64=True, supports_atomics=True, warp_size=info.warp_size,
            max_registers_per_block=info.max_registers_per_block, clock_rate_khz=info.clock_rate_khz,
            multiprocessor_count=info.multiprocessor_count, is_cpu=False)

    _devices = None

    @classmethod
    def init(cls):
        """Device.init: enumerate; an unavailable backend gives no devices rather than an error."""
        cls._devices = []
        if hip.lib.sarek_hip_is_available():
            n = C.c_int(0)
            hip.check(hip.lib.sarek_hip_device_count(C.byref(n)))
            cls._devices = [cls(i, hip.device_info(i)) for i in range(n.value)]
        return cls._devices

    @classmethod
    def all(cls):
        return cls._devices if cls._devices is not None else cls.init()

    @classmethod
    def count(cls):
        return len(cls.all())

    @classmethod
    def get(cls, dev_id):
        devs = cls.all()
        return devs[dev_id] if 0 <= dev_id < len(devs) else None

    @classmethod
    def first(cls):
        return cls.get(0)

    best = first

    @classmethod
    def by_framework(cls, framework):
        return [d for d in cls.all() if d.framework == framework]

    @classmethod
    def reset(cls):
        cls._devices = None

    def to_string(self):
        major, minor = self.capabilities["compute_capability"]
        sm = f"SM {major}.{minor}" if major > 0 else self.framework
        return (f"[{self.id}] {self.name} ({self.framework}) - {sm}, "
                f"{self.capabilities['total_global_mem'] / 2 ** 30:.1f} GB, {self.capabilities['multiprocessor_count']} MPs")

    __str__ = to_string

    is_gpu, is_cpu = True, False

    def __getattr__(self, name):            # warp_size, max_threads_per_block, multiprocessor_count, ...
        caps = self.__dict__.get("capabilities", {})
        if name in caps:
            return caps[name]
        raise AttributeError(name)

    @property
    def total_memory(self):
        return self.capabilities["total_global_mem"]

    @property
    def allows_fp64(self):
        return self.capabilities["supports_fp64"]

    def free_memory(self):
        self.set_current()
        free, total = C.c_size_t(0), C.c_size_t(0)
        hip.check(hip.lib.sarek_hip_mem_get_info(C.byref(free), C.byref(total)))
        return free.value

    def set_current(self):
        hip.check(hip.lib.sarek_hip_device_set_current(self.id))

    def synchronize(self):
        self.set_current()
        hip.check(hip.lib.sarek_hip_device_synchronize())


class _Kind:
    def __init__(self, code, name, dtype):
        self.code, self.name, self.dtype = code, name, np.dtype(dtype) if dtype is not None else None

    def __repr__(self):
        return self.name


class Vector:
    """sarek/core/Vector.ml; a host block, per-device buffers, a location."""
    float32 = _Kind(0, "Float32", np.float32)
    float64 = _Kind(1, "Float64", np.float64)
    int32 = _Kind(2, "Int32", np.int32)
    int64 = _Kind(3, "Int64", np.int64)
    char = _Kind(4, "Char", np.uint8)
    complex32 = _Kind(5, "Complex32", np.complex64)

    def __init__(self, handle, kind):
        self._h, self._kind = handle, kind

    # -- kinds (Vector_types.elem_size / kind_name) --
    @staticmethod
    def elem_size(kind):
        return kind.dtype.itemsize

    @staticmethod
    def kind_name(kind):
        return kind.name

    @classmethod
    def create_float32(cls, length): return cls.create(cls.float32, length)

    @classmethod
    def create_float64(cls, length): return cls.create(cls.float64, length)

    @classmethod
    def create_int32(cls, length): return cls.create(cls.int32, length)

    @classmethod
    def create_int64(cls, length): return cls.create(cls.int64, length)

    # -- creation (Vector_storage.create / create_custom / of_array) --
    @classmethod
    def create(cls, kind, length, pinned=False, zero_copy=False):
        """pinned: host block from pinned memory (copies run at the full link rate, no staging).
        zero_copy: pinned, and the device works on the host block itself: no copies at all."""
        h = C.c_void_p()
        hip.check(hip.lib.sarek_hip_vector_create(kind.code, length, 0, 2 if zero_copy else int(pinned), C.byref(h)))
        return cls(h, kind)

    @classmethod
    def create_custom(cls, elem_size, length, pinned=False):
        h = C.c_void_p()
        hip.check(hip.lib.sarek_hip_vector_create(6, length, elem_size, int(pinned), C.byref(h)))
        return cls(h, _Kind(6, f"Custom({elem_size})", np.dtype((np.void, elem_size))))

    @classmethod
    def of_array(cls, array, kind=None, pinned=False):
        array = np.ascontiguousarray(array)
        kind = kind or next(k for k in (cls.float32, cls.float64, cls.int32, cls.int64, cls.char, cls.complex32)
                            if k.dtype == array.dtype)
        v = cls.create(kind, array.size, pinned)
        v.host[:] = array.reshape(-1).astype(kind.dtype, copy=False)      # straight into the host block: stays CPU
        return v

    @classmethod
    def of_list(cls, kind, values):
        """Vector.of_list kind l."""
        return cls.of_array(np.asarray(list(values), dtype=kind.dtype), kind)

    @classmethod
    def of_bigarray(cls, kind, array):
        """Vector.of_bigarray: a numpy array stands in for the Bigarray; the vector gets a block of its own."""
        return cls.of_array(array, kind)

    def to_bigarray(self):
        """Vector.to_bigarray: the host block itself, no sync (Vector.ml:57-62)."""
        if self._kind.code == 6:
            raise ValueError("to_bigarray: vector uses custom storage")
        return self.host

    @classmethod
    def init(cls, kind, length, f):
        """Vector.init kind n f."""
        v = cls.create(kind, length)
        v.host[:] = np.fromiter((f(i) for i in range(length)), dtype=kind.dtype, count=length)
        return v

    def fill(self, value):
        """Vector.fill: the host block, then the bookkeeping of a host write."""
        elem = np.asarray([value], dtype=self._kind.dtype)
        hip.check(hip.lib.sarek_hip_vector_fill(self._h, C.c_void_p(elem.ctypes.data)))

    def copy(self):
        """Vector.copy: host data only (downloaded first if stale), location CPU."""
        h = C.c_void_p()
        hip.check(hip.lib.sarek_hip_vector_copy(self._h, C.byref(h)))
        return Vector(h, self._kind)

    def sub_vector(self, start, length, ok_range=None, ko_range=0):
        """Vector.sub_vector vec ~start ~len ?ok_range ?ko_range (): shares the host block."""
        h = C.c_void_p()
        st = hip.lib.sarek_hip_vector_sub(self._h, start, length, -1 if ok_range is None else ok_range, ko_range,
                                          C.byref(h))
        if st == hip.E_INVALID_ARG:
            raise IndexError(hip.lib.sarek_hip_last_error().decode())      # Invalid_argument in the reference
        hip.check(st)
        return Vector(h, self._kind)

    def partition(self, devices):
        """Vector.partition vec devices: one sub-vector per device id, each Stale_GPU of its device."""
        n = len(devices)
        out = (C.c_void_p * max(n, 1))()
        hip.check(hip.lib.sarek_hip_vector_partition(self._h, n, (C.c_int * max(n, 1))(*devices), out))
        return [Vector(C.c_void_p(out[i]), self._kind) for i in range(n)]

    @staticmethod
    def blit(src, src_off, dst, dst_off, length):
        st = hip.lib.sarek_hip_vector_blit(src._h, src_off, dst._h, dst_off, length)
        if st == hip.E_INVALID_ARG:
            raise IndexError(hip.lib.sarek_hip_last_error().decode())
        hip.check(st)

    def _sub_meta(self):
        is_sub, depth = C.c_int(0), C.c_int(0)
        parent, start, ok, ko = C.c_int64(0), C.c_int64(0), C.c_int64(0), C.c_int64(0)
        hip.check(hip.lib.sarek_hip_vector_sub_meta(self._h, C.byref(is_sub), C.byref(parent), C.byref(start),
                                                    C.byref(ok), C.byref(ko), C.byref(depth)))
        return bool(is_sub.value), parent.value, start.value, ok.value, ko.value, depth.value

    @property
    def id(self):
        return hip.lib.sarek_hip_vector_id(self._h)

    @property
    def is_sub(self):
        return self._sub_meta()[0]

    @property
    def depth(self):
        return self._sub_meta()[5]

    @property
    def parent_id(self):
        m = self._sub_meta()
        return m[1] if m[0] else None

    @property
    def sub_start(self):
        m = self._sub_meta()
        return m[2] if m[0] else None

    @property
    def sub_ok_range(self):
        m = self._sub_meta()
        return m[3] if m[0] else None

    @property
    def sub_ko_range(self):
        m = self._sub_meta()
        return m[4] if m[0] else None

    # location queries (Vector.ml:154-172)
    @property
    def is_on_cpu(self):
        return self.location in (CPU, Both, Stale_GPU)

    @property
    def is_on_gpu(self):
        return self.location in (GPU, Both, Stale_CPU)

    @property
    def is_synced(self):
        return self.location == Both

    @property
    def needs_gpu_update(self):
        return self.location == Stale_GPU

    @property
    def needs_cpu_update(self):
        return self.location in (Stale_CPU, GPU)

    def __str__(self):
        buf = C.create_string_buffer(256)
        hip.check(hip.lib.sarek_hip_vector_to_string(self._h, buf, 256))
        return buf.value.decode()

    def destroy(self):
        if self._h is not None:
            hip.check(hip.lib.sarek_hip_vector_destroy(self._h))
            self._h = None

    def __del__(self):                  # the reference frees device buffers from a GC finaliser
        try:
            self.destroy()
        except Exception:
            pass

    # -- accessors --
    @property
    def length(self):
        return hip.lib.sarek_hip_vector_length(self._h)

    def __len__(self):
        return self.length

    @property
    def kind(self):
        return self._kind

    @property
    def location(self):
        loc = C.c_int(0)
        hip.check(hip.lib.sarek_hip_vector_location(self._h, C.byref(loc), None))
        return _LOCATIONS[loc.value]

    @property
    def host(self):
        """The raw host block as a numpy view (Vector.host_ptr): no sync, no location update."""
        n = self.length
        ptr = hip.lib.sarek_hip_vector_host_ptr(self._h)
        if n == 0:
            return np.empty(0, dtype=self._kind.dtype)
        buf = (C.c_char * (n * self._kind.dtype.itemsize)).from_address(ptr)
        return np.frombuffer(buf, dtype=self._kind.dtype, count=n)

    @property
    def device_ptr(self):
        p = C.c_void_p()
        hip.check(hip.lib.sarek_hip_vector_device_ptr(self._h, C.byref(p)))
        return p.value

    def set_auto_sync(self, enabled):
        hip.check(hip.lib.sarek_hip_vector_set_auto_sync(self._h, int(enabled)))

    @property
    def auto_sync(self):
        return bool(hip.lib.sarek_hip_vector_auto_sync(self._h))

    # -- element access (Vector.get / Vector.set) --
    def get(self, index):
        out = np.empty(1, dtype=self._kind.dtype)
        st = hip.lib.sarek_hip_vector_get(self._h, index, C.c_void_p(out.ctypes.data))
        if st == hip.E_INVALID_ARG:
            raise IndexError(hip.lib.sarek_hip_last_error().decode())      # Invalid_argument in the reference
        hip.check(st)
        return out[0]

    def set(self, index, value):
        elem = np.asarray([value], dtype=self._kind.dtype)
        st = hip.lib.sarek_hip_vector_set(self._h, index, C.c_void_p(elem.ctypes.data))
        if st == hip.E_INVALID_ARG:
            raise IndexError(hip.lib.sarek_hip_last_error().decode())
        hip.check(st)

    __getitem__ = get
    __setitem__ = set

    def unsafe_get(self, index):
        """Vector.unsafe_get: the host block as it is -- no bounds check, no sync (Vector.ml:118-122)."""
        return self.host[index]

    def unsafe_set(self, index, value):
        """Vector.unsafe_set: no bounds check; the location follows as for set (Vector.ml:124-133)."""
        self.set(index, value)

    # -- the element-wise conveniences (Vector.ml:318-470): each syncs the host copy first, then works on it --
    def iter(self, f):
        for x in self.to_array():
            f(x)

    def iteri(self, f):
        for i, x in enumerate(self.to_array()):
            f(i, x)

    def map(self, f, kind):
        return Vector.of_array(np.asarray([f(x) for x in self.to_array()], dtype=kind.dtype), kind)

    def mapi(self, f, kind):
        return Vector.of_array(np.asarray([f(i, x) for i, x in enumerate(self.to_array())], dtype=kind.dtype), kind)

    def map_inplace(self, f):
        self.fill_from(np.asarray([f(x) for x in self.to_array()], dtype=self._kind.dtype))

    def fold_left(self, f, init):
        acc = init
        for x in self.to_array():
            acc = f(acc, x)
        return acc

    def fold_right(self, f, init):
        acc = init
        for x in self.to_array()[::-1]:
            acc = f(x, acc)
        return acc

    def for_all(self, p):
        return all(p(x) for x in self.to_array())

    def exists(self, p):
        return any(p(x) for x in self.to_array())

    def find(self, p):
        return next((x for x in self.to_array() if p(x)), None)

    def find_index(self, p):
        return next((i for i, x in enumerate(self.to_array()) if p(x)), None)

    def sum(self, zero, add):
        return self.fold_left(add, zero)

    def min_elt(self, compare):
        a = self.to_array()
        if a.size == 0:
            return None
        m = a[0]
        for x in a[1:]:
            if compare(x, m) < 0:
                m = x
        return m

    def max_elt(self, compare):
        a = self.to_array()
        if a.size == 0:
            return None
        m = a[0]
        for x in a[1:]:
            if compare(x, m) > 0:
                m = x
        return m

    def to_list(self):
        return list(self.to_array())

    def to_array(self):
        """Vector.to_array: a fresh array; downloads first when the host copy is stale."""
        out = np.empty(self.length, dtype=self._kind.dtype)
        hip.check(hip.lib.sarek_hip_vector_read(self._h, C.c_void_p(out.ctypes.data), 0, out.size))
        return out

    def fill_from(self, array, first=0):
        """A loop of Vector.set over a range, in one call."""
        array = np.ascontiguousarray(array, dtype=self._kind.dtype)
        st = hip.lib.sarek_hip_vector_write(self._h, C.c_void_p(array.ctypes.data), first, array.size)
        if st == hip.E_INVALID_ARG:
            raise IndexError(hip.lib.sarek_hip_last_error().decode())
        hip.check(st)


class GpuMemory:
    """sarek/core/Gpu_memory.ml over the library's counters: the native Vector layer tracks every device buffer it
    allocates and frees, and allocates through with_retry; Python's collector is the reclaim callback."""

    class Stats(C.Structure):
        _fields_ = [(n, C.c_int64) for n in ("current_bytes", "peak_bytes", "alloc_count", "free_count",
                                              "gc_free_count", "gc_freed_bytes", "retry_count")]

    _ATTEMPT = C.CFUNCTYPE(C.c_int, C.c_void_p)
    _RECLAIM = C.CFUNCTYPE(None, C.c_void_p, C.c_int)
    _reclaim = None

    @staticmethod
    def set_auto_gc(enabled): hip.lib.sarek_hip_gpu_memory_set_auto_gc(int(enabled))

    @staticmethod
    def get_auto_gc(): return bool(hip.lib.sarek_hip_gpu_memory_get_auto_gc())

    @staticmethod
    def track_alloc(nbytes): hip.lib.sarek_hip_gpu_memory_track_alloc(nbytes)

    @staticmethod
    def track_free(nbytes): hip.lib.sarek_hip_gpu_memory_track_free(nbytes)

    @staticmethod
    def usage(): return hip.lib.sarek_hip_gpu_memory_usage()

    @staticmethod
    def peak_usage(): return hip.lib.sarek_hip_gpu_memory_peak_usage()

    @classmethod
    def stats(cls):
        s = cls.Stats()
        hip.check(hip.lib.sarek_hip_gpu_memory_stats(C.byref(s)))
        return s

    @staticmethod
    def reset_stats(): hip.lib.sarek_hip_gpu_memory_reset_stats()

    @staticmethod
    def trigger_gc(): hip.lib.sarek_hip_gpu_memory_trigger_gc()

    @classmethod
    def use_python_collector(cls):
        """Registers gc.collect() as what a retry runs between two attempts (Gc.full_major / Gc.compact there)."""
        import gc
        cls._reclaim = cls._RECLAIM(lambda ctx, attempt: gc.collect() and None)
        hip.lib.sarek_hip_gpu_memory_set_reclaim(C.cast(cls._reclaim, C.c_void_p), None)

    @classmethod
    def with_retry(cls, f):
        """Gpu_memory.with_retry f: f raises to fail; the first failure is the one re-raised after three."""
        box = {}

        def attempt(ctx):
            try:
                box["value"] = f()
                return 0
            except Exception as e:          # noqa: BLE001 -- any failure counts, as `with exn1` there
                box.setdefault("first", e)
                return hip.E_INVALID_ARG
        cb = cls._ATTEMPT(attempt)
        if hip.lib.sarek_hip_gpu_memory_with_retry(C.cast(cb, C.c_void_p), None) != 0:
            raise box["first"]
        return box["value"]


class Transfer:
    """sarek/core/Transfer.ml (the device is the current one)."""

    @staticmethod
    def to_device(vec):
        hip.check(hip.lib.sarek_hip_transfer_to_device(vec._h))

    @staticmethod
    def to_cpu(vec, force=False):
        hip.check(hip.lib.sarek_hip_transfer_to_cpu(vec._h, int(force)))

    @staticmethod
    def sync(vec):
        hip.check(hip.lib.sarek_hip_transfer_sync(vec._h))

    @staticmethod
    def free_all_buffers(vec):
        hip.check(hip.lib.sarek_hip_transfer_free_buffers(vec._h))

    @staticmethod
    def flush():
        hip.check(hip.lib.sarek_hip_transfer_flush())

    @staticmethod
    def set_auto(enabled):
        hip.check(hip.lib.sarek_hip_transfer_set_auto(int(enabled)))

    # batch operations and streams (Transfer.ml:392-452)
    @staticmethod
    def to_device_all(vecs):
        for v in vecs:
            Transfer.to_device(v)

    @staticmethod
    def to_cpu_all(vecs):
        for v in vecs:
            Transfer.to_cpu(v)

    @staticmethod
    def sync_all(vecs):
        for v in vecs:
            Transfer.sync(v)

    @staticmethod
    def create_stream():
        s = C.c_void_p()
        hip.check(hip.lib.sarek_hip_stream_create(C.byref(s)))
        return s

    @staticmethod
    def default_stream():
        return C.c_void_p(None)

    @staticmethod
    def synchronize_stream(stream):
        hip.check(hip.lib.sarek_hip_stream_synchronize(stream))

    @staticmethod
    def destroy_stream(stream):
        if stream is not None and stream.value:          # the default stream is never destroyed
            hip.check(hip.lib.sarek_hip_stream_destroy(stream))


class Execute:
    """sarek/sarek/Execute.ml: vector_arg constructors, run_vectors, run_source."""

    @staticmethod
    def Vec(v): return ("vec", v)
    @staticmethod
    def Int(n): return ("i32", int(n))          # expand_to_run_source_args sends Int as Int32
    @staticmethod
    def Int32(n): return ("i32", int(n))
    @staticmethod
    def Int64(n): return ("i64", int(n))
    @staticmethod
    def Float32(x): return ("f32", float(x))
    @staticmethod
    def Float64(x): return ("f64", float(x))

    @staticmethod
    def dims1d(x): return (x, 1, 1)
    @staticmethod
    def dims2d(x, y): return (x, y, 1)
    @staticmethod
    def dims3d(x, y, z): return (x, y, z)

    @staticmethod
    def grid_for_size(problem_size, block_size):
        return (problem_size + block_size - 1) // block_size

    @staticmethod
    def grid_for(problem_size, block_size):
        return Execute.dims1d(Execute.grid_for_size(problem_size, block_size))

    @staticmethod
    def supports_lang(lang):
        return bool(hip.lib.sarek_hip_supports_lang(lang))

    @staticmethod
    def load_source(path):
        with open(path) as f:
            return f.read()

    @staticmethod
    def detect_lang(path):
        lang = C.c_int(0)
        st = hip.lib.sarek_hip_execute_detect_lang(str(path).encode(), C.byref(lang))
        if st == hip.E_INVALID_ARG:
            raise ValueError(hip.lib.sarek_hip_last_error().decode())      # Execution_error (Invalid_file ...)
        hip.check(st)
        return lang.value

    @staticmethod
    def run_source_file(path, kernel_name, block, grid, args, shared_mem=0, inject_lengths=True):
        a, n = Execute._args(args)
        hip.check(hip.lib.sarek_hip_execute_run_source_file(str(path).encode(), kernel_name.encode(),
                                                            (C.c_int * 3)(*block), (C.c_int * 3)(*grid), shared_mem,
                                                            int(inject_lengths), a, n))
        return hip.lib.sarek_hip_last_run_path().decode()

    @staticmethod
    def _args(args):
        out = (hip.VArg * max(len(args), 1))()
        for a, (kind, v) in zip(out, args):
            if kind == "vec":
                a.kind, a.vec = 0, v._h
            elif kind == "i32":
                a.kind, a.i32 = 1, v
            elif kind == "i64":
                a.kind, a.i64 = 2, v
            elif kind == "f32":
                a.kind, a.f32 = 3, v
            elif kind == "f64":
                a.kind, a.f64 = 4, v
            else:
                raise ValueError(f"unknown vector_arg {kind!r}")
        return out, len(args)

    @staticmethod
    def run_vectors(ir, args, block, grid, shared_mem=0):
        """Execute.run_vectors ~ir ~args ~block ~grid ?shared_mem (); returns the code path that
        served the launch ("jit" or a hand kernel's tag)."""
        a, n = Execute._args(args)
        hip.check(hip.lib.sarek_hip_execute_run_vectors(ir.encode(), (C.c_int * 3)(*block), (C.c_int * 3)(*grid),
                                                        shared_mem, a, n))
        return hip.lib.sarek_hip_last_run_path().decode()

    @staticmethod
    def run_pipeline(stages):
        """A kernel list run in order: stages = [(ir, args, block, grid)] or [(ir, args, block, grid, shared_mem)],
        each what one run_vectors call takes.  Returns (code paths, device launches made); consecutive stages
        that one hand kernel serves count as one launch."""
        arr = (hip.PipelineStage * max(len(stages), 1))()
        keep = []
        for st, stage in zip(arr, stages):
            ir, args, block, grid = stage[:4]
            a, n = Execute._args(args)
            text = ir.encode()
            keep.append((a, text))
            st.ir_text, st.block, st.grid = text, (C.c_int * 3)(*block), (C.c_int * 3)(*grid)
            st.shared_mem_bytes = stage[4] if len(stage) > 4 else 0
            st.args, st.n_args = a, n
        launches = C.c_int(0)
        hip.check(hip.lib.sarek_hip_execute_run_pipeline(arr, len(stages), C.byref(launches)))
        return hip.lib.sarek_hip_last_run_path().decode(), launches.value

    @staticmethod
    def library_kernel(name):
        """(source, kernel_name) of one of the backend's library kernels, to hand to run_source."""
        return hip.library_kernel(name)

    @staticmethod
    def run_source(source, kernel_name, block, grid, args, lang=hip.LANG_HIP, shared_mem=0, inject_lengths=True):
        a, n = Execute._args(args)
        hip.check(hip.lib.sarek_hip_execute_run_source(source.encode(), lang, kernel_name.encode(),
                                                       (C.c_int * 3)(*block), (C.c_int * 3)(*grid), shared_mem,
                                                       int(inject_lengths), a, n))
        return hip.lib.sarek_hip_last_run_path().decode()

    @staticmethod
    def sync_vectors_to_cpu(args):
        a, n = Execute._args(args)
        hip.check(hip.lib.sarek_hip_execute_sync_vectors_to_cpu(a, n))
