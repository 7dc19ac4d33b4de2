"""ctypes binding of libmi355_int8.so (the C ABI in include/mi355_int8.h).

Host-side plumbing for tests, smoke and the benchmark: it owns no arithmetic.
Device buffers come from the library's own arena (the device analog of the
upstream NumaArena, threading/numa_arena.mojo:5-87), so a test reads like the
upstream ones: make an arena, alloc, launch, wait, check
(test_linux_threading.mojo:164-215).

There is no CPU fallback: if the shared library is missing, import fails.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# MI355_INT8_LIB names another build of the same library (bench.py --gemm-timeline loads the instrumented one)
LIB_PATH = os.environ.get("MI355_INT8_LIB") or os.path.join(_HERE, "libmi355_int8.so")

OK, EIO, ENOMEM, EBUSY, ENODEV, EINVAL, ENOSPC, ERANGE = 0, -5, -12, -16, -19, -22, -28, -34

if not os.path.exists(LIB_PATH):
    raise ImportError(
        "libmi355_int8.so is not built (%s). Run `python -c 'import __graft_entry__ as g; g.build()'` "
        "or `make -C mojo-linuxperiments_amd/csrc`; there is no CPU fallback." % LIB_PATH)

lib = C.CDLL(LIB_PATH)

i32, i64, vp, f32p = C.c_int32, C.c_int64, C.c_void_p, C.POINTER(C.c_float)

# name -> (restype, argtypes); the same list drives the export check in tests
SIGNATURES = {
    "mi_status_string": (C.c_char_p, [i32]),
    "mi_last_hip_error": (i32, []),
    "mi_abi_version": (i32, []),
    "mi_ctx_create": (i32, [i32, C.POINTER(vp)]),
    "mi_ctx_destroy": (i32, [vp]),
    "mi_ctx_device": (i32, [vp]),
    "mi_ctx_compute_units": (i32, [vp]),
    "mi_ctx_memory_bytes": (i64, [vp]),
    "mi_ctx_arch_name": (i32, [vp, C.c_char_p, i64]),
    "mi_arena_create": (i32, [vp, i64, i64, C.POINTER(vp)]),
    "mi_host_arena_create": (i32, [vp, i64, i64, i32, C.POINTER(vp)]),
    "mi_arena_destroy": (i32, [vp]),
    "mi_arena_alloc": (vp, [vp, i64]),
    "mi_arena_mark": (i64, [vp]),
    "mi_arena_reset_to": (i32, [vp, i64]),
    "mi_arena_reset": (i32, [vp]),
    "mi_arena_remaining": (i64, [vp]),
    "mi_arena_used": (i64, [vp]),
    "mi_arena_verify_placement": (i32, [vp]),
    "mi_stream_pool_create": (i32, [vp, i32, C.POINTER(vp)]),
    "mi_stream_pool_destroy": (i32, [vp]),
    "mi_stream_pool_capacity": (i32, [vp]),
    "mi_stream_pool_begin": (i32, [vp]),
    "mi_stream_pool_stream": (vp, [vp, i32]),
    "mi_stream_pool_end": (i32, [vp, i32]),
    "mi_stream_pool_in_use": (i32, [vp, i32]),
    "mi_stream_pool_wait_all": (i32, [vp]),
    "mi_stream_pool_wait_any": (i32, [vp]),
    "mi_gate_create": (i32, [vp, C.POINTER(vp)]),
    "mi_gate_destroy": (i32, [vp]),
    "mi_gate_release": (i32, [vp, vp]),
    "mi_gate_wait": (i32, [vp, vp]),
    "mi_gate_wait_host": (i32, [vp]),
    "mi_gate_reset": (i32, [vp]),
    "mi_graph_capture_begin": (i32, [vp]),
    "mi_graph_capture_end": (i32, [vp, C.POINTER(vp)]),
    "mi_graph_launch": (i32, [vp, vp]),
    "mi_graph_destroy": (i32, [vp]),
    "mi_memcpy_h2d": (i32, [vp, vp, i64, vp]),
    "mi_memcpy_d2h": (i32, [vp, vp, i64, vp]),
    "mi_memcpy_d2d": (i32, [vp, vp, i64, vp]),
    "mi_fill_u32": (i32, [vp, C.c_uint32, i64, vp]),
    "mi_stream_synchronize": (i32, [vp]),
    "mi_host_alloc": (vp, [i64]),
    "mi_host_free": (i32, [vp]),
    "mi_event_create": (i32, [C.POINTER(vp)]),
    "mi_event_destroy": (i32, [vp]),
    "mi_event_record": (i32, [vp, vp]),
    "mi_event_synchronize": (i32, [vp]),
    "mi_event_elapsed_ms": (i32, [vp, vp, f32p]),
    "mi_fwht_quant_f32_i8": (i32, [vp, vp, vp, i64, i64, i32, vp]),
    "mi_fwht_quant_batch_f32_i8": (i32, [vp, i32, i32, vp]),
    "mi_fwht_f32": (i32, [vp, vp, i64, i64, i32, vp]),
    "mi_w8a8_gemm_i32": (i32, [vp, vp, vp, i64, i64, i64, vp]),
    "mi_w8a8_gemm_dequant_f32": (i32, [vp, vp, vp, vp, vp, i64, i64, i64, vp]),
    "mi_dequant_i32_f32": (i32, [vp, vp, vp, vp, i64, i64, vp]),
    "mi_gemm_batch_plan_bytes": (i64, [vp, i32]),
    "mi_gemm_batch_plan_host": (i64, [vp, i32, i32, vp, i64, C.POINTER(i32)]),
    "mi_gemm_batch_create": (i32, [vp, i32, vp, i64, C.POINTER(vp)]),
    "mi_gemm_batch_destroy": (i32, [vp]),
    "mi_gemm_batch_run_f32": (i32, [vp, vp, vp]),
    "mi_gemm_batch_run_i32": (i32, [vp, vp, vp]),
    "mi_w8a8_linear_workspace_bytes": (i64, [i64, i64, i64]),
    "mi_w8a8_linear_f32": (i32, [vp, vp, vp, vp, i64, i64, i64, i32, vp, i64, vp]),
    "mi_w8a8_linear_f32_noalloc": (i32, [vp, vp, vp, vp, i64, i64, i64, i32, vp]),
    "mi_w8a8_linear_noalloc_max_rows": (i64, []),
    "mi_w8a8_linear_noalloc_max_codes": (i64, []),
    "mi_gqa_decode_workspace_bytes": (i64, [i64, i64, i64, i64, i64]),
    "mi_gqa_decode_attn": (i32, [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i32, vp, i64, vp]),
    "mi_gqa_decode_attn_cache": (i32, [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, vp, i64, i32, vp, i64, vp]),
    "mi_rmsnorm_f32": (i32, [vp, vp, vp, C.c_float, vp, vp, i64, i64, vp]),
    "mi_rope_kv_append_f32_i8": (i32, [vp, i64, vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, vp]),
    "mi_swiglu_f32": (i32, [vp, vp, i64, i64, vp]),
    "mi_rmsnorm_quant_f32_i8": (i32, [vp, vp, vp, C.c_float, vp, vp, vp, vp, i64, i64, i32, vp]),
    "mi_rmsnorm_linear_f32": (i32, [vp, vp, vp, C.c_float, vp, vp, vp, vp, vp, i64, i64, i64, i32, vp, i64, vp]),
    "mi_swiglu_quant_f32_i8": (i32, [vp, vp, vp, vp, i64, i64, i32, vp]),
    "mi_add_f32": (i32, [vp, vp, vp, i64, vp]),
    "mi_gqa_decode_attn_cache_quant_i8": (i32, [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, vp, i64, vp,
                                                i64, vp]),
    "mi_gqa_decode_attn_paged": (i32, [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, vp, i64, i32, vp, i64,
                                       vp]),
    "mi_kv_append_paged_f32_i8": (i32, [vp, vp, i64, vp, vp, vp, vp, vp, i64, i64, vp, i64, i64, i64, vp]),
    "mi_kv_append_f32_i8": (i32, [vp, vp, i64, vp, vp, vp, vp, vp, i64, i64, i64, i64, vp]),
    "mi_gqa_decode_attn_tiled": (i32, [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, vp, i64, i32, vp, i64, vp]),
    "mi_gqa_decode_attn_linear_workspace_bytes": (i64, [i64, i64, i64, i64, i64]),
    "mi_gqa_decode_attn_tiled_linear_f32": (i32, [vp, vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, vp, i64, i64,
                                                  vp, i64, vp]),
    "mi_gqa_decode_attn_tiled_quant_i8": (i32, [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, vp, i64, vp, i64,
                                             vp]),
    "mi_kv_tiled_from_rows_i8": (i32, [vp, vp, vp, vp, i64, i64, i64, i64, vp]),
    "mi_kv_append_tiled_f32_i8": (i32, [vp, vp, i64, vp, vp, vp, vp, vp, i64, i64, i64, i64, vp]),
    "mi_rope_kv_append_tiled_f32_i8": (i32, [vp, i64, vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, vp]),
    "mi_gqa_decode_attn_tiled_paged": (i32, [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, vp, i64, i32, vp, i64, vp]),
    "mi_gqa_decode_attn_tiled_paged_quant_i8": (i32, [vp, vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, vp, i64,
                                                       vp, i64, vp]),
    "mi_kv_append_tiled_paged_f32_i8": (i32, [vp, vp, i64, vp, vp, vp, vp, vp, i64, vp, i64, i64, i64, vp]),
    "mi_rope_kv_append_tiled_paged_f32_i8": (i32, [vp, i64, vp, vp, vp, vp, vp, vp, vp, vp, i64, vp, i64, i64, i64, i64, vp]),
    "mi_gqa_decode_scores_tiled_i32": (i32, [vp] * 8 + [i64, i64, i64, i64, i64, i64, vp, i64, vp]),
    "mi_gqa_decode_scores_i32": (i32, [vp] * 8 + [i64, i64, i64, i64, i64, vp, i64, vp]),
    "mi_moe_route_workspace_bytes": (i64, [i64, i64]),
    "mi_moe_route": (i32, [vp, vp, vp, vp, i64, i64, i64, i32, vp, i64, vp]),
    "mi_moe_dispatch": (i32, [vp, vp, vp, i64, i64, i32, vp]),
    "mi_moe_ffn_workspace_bytes": (i64, [i64, i64, i64, i64, i32]),
    "mi_moe_ffn": (i32, [vp] * 10 + [i64, i64, i64, i64, i32, vp, i64, vp]),
    "mi_moe_ffn_workspace_offset": (i64, [i32, i64, i64, i64, i64, i32]),
    "mi_moe_layer": (i32, [vp] * 9 + [i64, i64, i64, i64, i32, vp, i64, vp]),
    "mi_moe_layer_workspace_bytes": (i64, [i64, i64, i64, i64, i32]),
}

_missing = []
for _name, (_res, _args) in SIGNATURES.items():
    try:
        _fn = getattr(lib, _name)
    except AttributeError:
        _missing.append(_name)
        continue
    _fn.restype = _res
    _fn.argtypes = _args
if _missing:
    raise ImportError("libmi355_int8.so lacks symbols: %s" % ", ".join(_missing))


class MiError(RuntimeError):
    def __init__(self, status, what=""):
        self.status = status
        msg = lib.mi_status_string(status).decode()
        if status == EIO:
            msg += " (hipError %d)" % lib.mi_last_hip_error()
        super().__init__("%s: %s [%d]" % (what, msg, status))


def check(status, what=""):
    if status != OK:
        raise MiError(status, what)


class DevBuf:
    """A typed view of arena memory: device pointer + shape + dtype."""

    def __init__(self, ptr, shape, dtype):
        self.ptr = ptr
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)

    @property
    def nbytes(self):
        return int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize

    def offset(self, nbytes, shape, dtype):
        return DevBuf(self.ptr + int(nbytes), shape, dtype)


class Device:
    """Context + one device arena + upload / download helpers."""

    def __init__(self, device=0, arena_bytes=1 << 30, alignment=256):
        self.ctx = vp()
        check(lib.mi_ctx_create(device, C.byref(self.ctx)), "mi_ctx_create")
        self.arena = vp()
        rc = lib.mi_arena_create(self.ctx, arena_bytes, alignment, C.byref(self.arena))
        if rc != OK:
            lib.mi_ctx_destroy(self.ctx)
            raise MiError(rc, "mi_arena_create")

    def close(self):
        if self.arena:
            lib.mi_arena_destroy(self.arena)
            self.arena = None
        if self.ctx:
            lib.mi_ctx_destroy(self.ctx)
            self.ctx = None

    @property
    def compute_units(self):
        return lib.mi_ctx_compute_units(self.ctx)

    @property
    def arch(self):
        buf = C.create_string_buffer(64)
        check(lib.mi_ctx_arch_name(self.ctx, buf, 64))
        return buf.value.decode()

    def mark(self):
        return lib.mi_arena_mark(self.arena)

    def reset_to(self, mark):
        check(lib.mi_arena_reset_to(self.arena, mark), "mi_arena_reset_to")

    def empty(self, shape, dtype):
        shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        nbytes = int(np.prod(shape, dtype=np.int64)) * np.dtype(dtype).itemsize
        p = lib.mi_arena_alloc(self.arena, max(nbytes, 1))
        if not p:
            raise MiError(ENOMEM, "mi_arena_alloc(%d)" % nbytes)
        return DevBuf(p, shape, dtype)

    def upload(self, arr, stream=None):
        arr = np.ascontiguousarray(arr)
        b = self.empty(arr.shape, arr.dtype)
        check(lib.mi_memcpy_h2d(b.ptr, arr.ctypes.data, arr.nbytes, stream), "mi_memcpy_h2d")
        check(lib.mi_stream_synchronize(stream))
        return b

    def download(self, buf, stream=None):
        out = np.empty(buf.shape, buf.dtype)
        check(lib.mi_stream_synchronize(stream))
        check(lib.mi_memcpy_d2h(out.ctypes.data, buf.ptr, out.nbytes, stream), "mi_memcpy_d2h")
        check(lib.mi_stream_synchronize(stream))
        return out

    def sync(self, stream=None):
        check(lib.mi_stream_synchronize(stream), "mi_stream_synchronize")


class Event:
    def __init__(self):
        self.h = vp()
        check(lib.mi_event_create(C.byref(self.h)), "mi_event_create")

    def record(self, stream=None):
        check(lib.mi_event_record(self.h, stream), "mi_event_record")

    def synchronize(self):
        check(lib.mi_event_synchronize(self.h), "mi_event_synchronize")

    def elapsed_ms(self, stop):
        ms = C.c_float()
        check(lib.mi_event_elapsed_ms(self.h, stop.h, C.byref(ms)), "mi_event_elapsed_ms")
        return float(ms.value)

    def destroy(self):
        if self.h:
            lib.mi_event_destroy(self.h)
            self.h = None


class StreamPool:
    """Fixed-capacity pool of streams; launch() mirrors ThreadPool.launch
    (threading/linux_threading.mojo:103-121): first free slot or False."""

    def __init__(self, dev, capacity):
        self.h = vp()
        check(lib.mi_stream_pool_create(dev.ctx, capacity, C.byref(self.h)), "mi_stream_pool_create")

    def stream(self, slot):
        return lib.mi_stream_pool_stream(self.h, slot)

    def launch(self, fn, *args):
        slot = lib.mi_stream_pool_begin(self.h)
        if slot < 0:
            return False
        fn(*args, stream=self.stream(slot))
        check(lib.mi_stream_pool_end(self.h, slot), "mi_stream_pool_end")
        return True

    def wait_all(self):
        check(lib.mi_stream_pool_wait_all(self.h), "mi_stream_pool_wait_all")

    def wait_any(self):
        return lib.mi_stream_pool_wait_any(self.h)

    def destroy(self):
        if self.h:
            check(lib.mi_stream_pool_destroy(self.h), "mi_stream_pool_destroy")
            self.h = None


class Graph:
    """Record the calls made inside `with Graph.capture(stream) as g:` and replay them."""

    def __init__(self, stream):
        self.stream = stream
        self.h = vp()

    @classmethod
    def capture(cls, stream):
        return cls(stream)

    def __enter__(self):
        check(lib.mi_graph_capture_begin(self.stream), "mi_graph_capture_begin")
        return self

    def __exit__(self, exc_type, exc, tb):
        rc = lib.mi_graph_capture_end(self.stream, C.byref(self.h))
        if exc_type is None:
            check(rc, "mi_graph_capture_end")
        return False

    def launch(self, stream=None):
        check(lib.mi_graph_launch(self.h, stream if stream is not None else self.stream), "mi_graph_launch")

    def destroy(self):
        if self.h:
            lib.mi_graph_destroy(self.h)
            self.h = None


# ---- thin checked wrappers over the kernel entry points (DevBuf in, status checked) ----

def fwht_quant(x, q, scale, block, stream=None):
    M, K = x.shape
    check(lib.mi_fwht_quant_f32_i8(x.ptr, q.ptr, scale.ptr, M, K, block, stream), "mi_fwht_quant_f32_i8")


class QuantRows(C.Structure):
    """mi_quant_rows of the header: one row set of a batched rotate + quantize call."""
    _fields_ = [("x", vp), ("q", vp), ("scale", vp), ("M", i64), ("K", i64)]


def fwht_quant_batch(sets, block, stream=None):
    """sets: [(x, q, scale)] DevBufs, x fp32 [M,K]: one launch for all of them."""
    arr = (QuantRows * len(sets))()
    for a, (x, q, scale) in zip(arr, sets):
        a.x, a.q, a.scale, a.M, a.K = x.ptr, q.ptr, scale.ptr, x.shape[0], x.shape[1]
    check(lib.mi_fwht_quant_batch_f32_i8(arr, len(sets), block, stream), "mi_fwht_quant_batch_f32_i8")


def fwht(x, out, block, stream=None):
    M, K = x.shape
    check(lib.mi_fwht_f32(x.ptr, out.ptr, M, K, block, stream), "mi_fwht_f32")


class GemmProblem(C.Structure):
    """mi_gemm_problem of the header: one contraction of a batch."""
    _fields_ = [("qx", vp), ("sx", vp), ("qw", vp), ("sw", vp), ("out", vp), ("M", i64), ("N", i64), ("K", i64)]


class GemmBatch:
    """Several W8A8 contractions in one launch (mi_gemm_batch_*): made once for a list of (M, N, K) shapes, run
    with the operands of each call.  The tile lists live in arena memory of `dev`."""

    def __init__(self, dev, shapes):
        self.shapes = [tuple(int(v) for v in s) for s in shapes]
        n = len(self.shapes)
        mnk = (i64 * (3 * n))(*[v for s in self.shapes for v in s])
        nbytes = lib.mi_gemm_batch_plan_bytes(mnk, n)
        if nbytes < 0:
            raise MiError(int(nbytes), "mi_gemm_batch_plan_bytes")
        self.plan = dev.empty(nbytes, np.uint8)
        self.h = vp()
        check(lib.mi_gemm_batch_create(mnk, n, self.plan.ptr, nbytes, C.byref(self.h)), "mi_gemm_batch_create")

    def _problems(self, ops):
        arr = (GemmProblem * len(ops))()
        for g, (qx, sx, qw, sw, out) in zip(arr, ops):
            g.qx, g.qw, g.out = qx.ptr, qw.ptr, out.ptr
            g.sx = sx.ptr if sx is not None else None
            g.sw = sw.ptr if sw is not None else None
            (g.M, g.K), g.N = qx.shape, qw.shape[0]
        return arr

    def run_f32(self, ops, stream=None):
        """ops: [(qx, sx, qw, sw, y)] DevBufs per problem."""
        check(lib.mi_gemm_batch_run_f32(self.h, self._problems(ops), stream), "mi_gemm_batch_run_f32")

    def run_i32(self, ops, stream=None):
        """ops: [(qx, None, qw, None, acc)] DevBufs per problem."""
        check(lib.mi_gemm_batch_run_i32(self.h, self._problems(ops), stream), "mi_gemm_batch_run_i32")

    def destroy(self):
        if self.h:
            lib.mi_gemm_batch_destroy(self.h)
            self.h = None


def gemm_i32(qx, qw, acc, stream=None):
    M, K = qx.shape
    N = qw.shape[0]
    check(lib.mi_w8a8_gemm_i32(qx.ptr, qw.ptr, acc.ptr, M, N, K, stream), "mi_w8a8_gemm_i32")


def gemm_dequant(qx, sx, qw, sw, y, stream=None):
    M, K = qx.shape
    N = qw.shape[0]
    check(lib.mi_w8a8_gemm_dequant_f32(qx.ptr, sx.ptr, qw.ptr, sw.ptr, y.ptr, M, N, K, stream),
          "mi_w8a8_gemm_dequant_f32")


def dequant(acc, sx, sw, y, stream=None):
    M, N = acc.shape
    check(lib.mi_dequant_i32_f32(acc.ptr, sx.ptr, sw.ptr, y.ptr, M, N, stream), "mi_dequant_i32_f32")


def linear(x, qw, sw, y, block, ws, stream=None):
    M, K = x.shape
    N = qw.shape[0]
    check(lib.mi_w8a8_linear_f32(x.ptr, qw.ptr, sw.ptr, y.ptr, M, N, K, block, ws.ptr, ws.nbytes, stream),
          "mi_w8a8_linear_f32")


def gqa_decode(q, kq, ks, vq, vs, o, out_rotated, ws, stream=None):
    B, Hq, D = q.shape
    _, Hkv, T, _ = kq.shape
    check(lib.mi_gqa_decode_attn(q.ptr, kq.ptr, ks.ptr, vq.ptr, vs.ptr, o.ptr, B, Hq, Hkv, D, T,
                                 1 if out_rotated else 0, ws.ptr, ws.nbytes, stream), "mi_gqa_decode_attn")


def gqa_scores(q, kq, ks, vq, vs, qq, sq, dots, ws, stream=None):
    B, Hq, D = q.shape
    _, Hkv, T, _ = kq.shape
    check(lib.mi_gqa_decode_scores_i32(q.ptr, kq.ptr, ks.ptr, vq.ptr, vs.ptr, qq.ptr, sq.ptr, dots.ptr,
                                       B, Hq, Hkv, D, T, ws.ptr, ws.nbytes, stream), "mi_gqa_decode_scores_i32")


def moe_route(x, wr, idx, w, topk, ws, stream=None):
    T, H = x.shape
    E = wr.shape[0]
    check(lib.mi_moe_route(x.ptr, wr.ptr, idx.ptr, w.ptr, T, H, E, topk, ws.ptr, ws.nbytes, stream), "mi_moe_route")


def moe_dispatch(idx, perm, seg, E, stream=None):
    T, topk = idx.shape
    check(lib.mi_moe_dispatch(idx.ptr, perm.ptr, seg.ptr, T, E, topk, stream), "mi_moe_dispatch")


def moe_ffn(x, idx, w, wg, sg, wu, su, wd, sd, y, ws, stream=None):
    T, H = x.shape
    E, I, _ = wg.shape
    topk = idx.shape[1]
    check(lib.mi_moe_ffn(x.ptr, idx.ptr, w.ptr, wg.ptr, sg.ptr, wu.ptr, su.ptr, wd.ptr, sd.ptr, y.ptr,
                         T, H, I, E, topk, ws.ptr, ws.nbytes, stream), "mi_moe_ffn")


def moe_layer(x, wr, wg, sg, wu, su, wd, sd, y, topk, ws, stream=None):
    T, H = x.shape
    E, I, _ = wg.shape
    check(lib.mi_moe_layer(x.ptr, wr.ptr, wg.ptr, sg.ptr, wu.ptr, su.ptr, wd.ptr, sd.ptr, y.ptr,
                           T, H, I, E, topk, ws.ptr, ws.nbytes, stream), "mi_moe_layer")


# ---- the matrix-pipe cache layouts restated in numpy (test and bench plumbing: what goes where) ----

def kv_rows_to_tiled(kq, vq, T_cap):
    """row-major codes [B,Hkv,T,128] -> kt [B,Hkv,T_cap/16,8,16,16] (chunk, token, byte) and
    vt [B,Hkv,T_cap/64,8,4,16,16] (dim piece, token chunk, dim, token); tokens past T are zero."""
    B, Hkv, T, D = kq.shape

    def pad(a):
        out = np.zeros((B, Hkv, T_cap, D), np.int8)
        out[:, :, :T] = a
        return out
    kt = np.ascontiguousarray(pad(kq).reshape(B, Hkv, T_cap // 16, 16, 8, 16).transpose(0, 1, 2, 4, 3, 5))
    vt = np.ascontiguousarray(pad(vq).reshape(B, Hkv, T_cap // 64, 4, 16, 8, 16).transpose(0, 1, 2, 5, 3, 6, 4))
    return kt, vt


def kv_tiled_to_rows(kt, vt):
    B, Hkv = kt.shape[:2]
    T_cap = kt.size // (B * Hkv * 128)
    kq = np.ascontiguousarray(kt.reshape(B, Hkv, T_cap // 16, 8, 16, 16).transpose(0, 1, 2, 4, 3, 5)).reshape(B, Hkv, T_cap, 128)
    vq = np.ascontiguousarray(vt.reshape(B, Hkv, T_cap // 64, 8, 4, 16, 16).transpose(0, 1, 2, 4, 6, 3, 5)).reshape(B, Hkv, T_cap, 128)
    return kq, vq


class DecoderLayer:
    """One decoder layer of a decode step, chained from the C-ABI entry points on one stream:
    (residual +) RMSNorm + quantize -> QKV GEMV -> rotary + KV-cache append -> attention over the cache (split,
    merge + quantize) -> O GEMV -> residual + RMSNorm + quantize -> gate|up GEMV -> SwiGLU + quantize -> down GEMV
    (-> residual).  Ten launches.  Test and bench plumbing over the same calls the C++ host struct of the same name makes
    (host/mi355_host.hpp).  trace=True also writes the fp32 rows the fused kernels normally keep in registers
    (xn, att, hn, act) so that a test can gate every stage."""

    def __init__(self, dev, B, H, Hq, Hkv, I, T_cap, wqkv, wo, wgu, wd, g1, g2, rope_cos, rope_sin, eps=1e-5,
                 block=128, trace=False, *, tiled, moe=None):
        """moe: None for the dense FFN (wgu, wd), or the experts of an MoE FFN in its place (wgu = wd = None):
        dict(wr fp32 [E,H], wg/wu int8 [E,I,H], sg/su fp32 [E,I], wd int8 [E,H,I], sd fp32 [E,H], topk), prepared codes.
        The second half of the layer is then residual + RMSNorm -> router, dispatch and grouped expert FFN ->
        residual."""
        D = 128
        self.moe = None
        # tiled (required, no default): the cache lives in the matrix-pipe layouts (capacity a multiple of 64 tokens)
        # or row-major; the layout never follows from the capacity
        self.tiled = bool(tiled)
        if self.tiled and T_cap % 64:
            raise MiError(EINVAL, "DecoderLayer: a tiled cache needs a capacity that is a multiple of 64 tokens")
        self.dev, self.B, self.H, self.Hq, self.Hkv, self.I, self.T_cap, self.eps, self.block = \
            dev, B, H, Hq, Hkv, I, T_cap, eps, block
        self.NQKV = (Hq + 2 * Hkv) * D

        def prep(w):
            N, K = w.shape
            q, s = dev.empty((N, K), np.int8), dev.empty(N, np.float32)
            keep = dev.mark()
            dw = dev.upload(w)
            fwht_quant(dw, q, s, block)
            dev.sync()
            dev.reset_to(keep)
            return q, s
        self.wqkv, self.wo = prep(wqkv), prep(wo)
        if moe is None:
            self.wgu, self.wd = prep(wgu), prep(wd)
        else:
            self.wgu = self.wd = None
            self.moe = {k: (dev.upload(v) if isinstance(v, np.ndarray) else v) for k, v in moe.items()}
            E = moe["wg"].shape[0]
            self.moe_ws = dev.empty(lib.mi_moe_layer_workspace_bytes(B, H, I, E, moe["topk"]), np.uint8)
        self.g1, self.g2 = dev.upload(g1), dev.upload(g2)
        self.cos, self.sin = dev.upload(rope_cos), dev.upload(rope_sin)
        self.kq, self.ks = dev.empty((B, Hkv, T_cap, D), np.int8), dev.empty((B, Hkv, T_cap), np.float32)
        self.vq, self.vs = dev.empty((B, Hkv, T_cap, D), np.int8), dev.empty((B, Hkv, T_cap), np.float32)
        f = np.float32
        self.h0, self.qkv = dev.empty((B, H), f), dev.empty((B, self.NQKV), f)
        self.q = dev.empty((B, Hq, D), f)
        self.att = dev.empty((B, Hq * D), f) if trace else None
        self.ca, self.sa = dev.empty((B, Hq * D), np.int8), dev.empty(B, f)   # codes of the attention rows
        self.ao, self.h1 = dev.empty((B, H), f), dev.empty((B, H), f)
        self.gu, self.dn = (dev.empty((B, 2 * I), f) if moe is None else None), dev.empty((B, H), f)
        self.xn = dev.empty((B, H), f) if trace else None
        self.hn = dev.empty((B, H), f) if (trace or moe is not None) else None   # the MoE FFN reads the normalized row
        self.act = dev.empty((B, I), f) if trace else None
        self.lin_ws = dev.empty(lib.mi_w8a8_linear_workspace_bytes(B, max(2 * I, self.NQKV), H), np.uint8)   # codes of the normalized rows
        self.ci, self.si = dev.empty((B, I), np.int8), dev.empty(B, f)        # codes of the activated rows
        self.att_ws = dev.empty(lib.mi_gqa_decode_attn_linear_workspace_bytes(B, Hq, Hkv, D, T_cap), np.uint8)
        if self.tiled:
            # the one-call attention + projection leaves the codes and scales of the attention rows in its workspace
            up = lambda v: (v + 255) // 256 * 256
            off = up(B * Hq * D * 4)
            self.ca = DevBuf(self.att_ws.ptr + off, (B, Hq * D), np.int8)
            self.sa = DevBuf(self.att_ws.ptr + off + up(B * Hq * D), (B,), f)

    def step(self, x, pos, seq_len, t_max, out, stream=None, residual=None):
        """x fp32 [B,H] (+ residual fp32 [B,H]: the layer input is their sum, left in self.h0); pos, seq_len int32
        [B] on the device (seq_len = pos + 1 for a plain decode step).  out fp32 [B,H], or None: the closing
        residual add is left to the next layer (pass x=self.dn, residual=self.h1 to its step)."""
        B, H, Hq, Hkv, I, D, s = self.B, self.H, self.Hq, self.Hkv, self.I, 128, stream
        p = lambda b: b.ptr if b is not None else None
        # norm + quantize + projection: one kernel for a single token, two launches otherwise
        check(lib.mi_rmsnorm_linear_f32(x.ptr, p(residual), self.g1.ptr, self.eps,
                                        self.h0.ptr if residual is not None else None, p(self.xn), self.wqkv[0].ptr,
                                        self.wqkv[1].ptr, self.qkv.ptr, B, self.NQKV, H, self.block, self.lin_ws.ptr,
                                        self.lin_ws.nbytes, s), "mi_rmsnorm_linear_f32")
        xin = self.h0 if residual is not None else x
        append = lib.mi_rope_kv_append_tiled_f32_i8 if self.tiled else lib.mi_rope_kv_append_f32_i8
        check(append(self.qkv.ptr, self.NQKV, self.cos.ptr, self.sin.ptr, self.q.ptr, self.kq.ptr, self.ks.ptr,
                     self.vq.ptr, self.vs.ptr, pos.ptr, B, Hq, Hkv, D, self.T_cap, s), "mi_rope_kv_append")
        # attention output stays in the rotated basis of V and is quantized by the merge itself: the O weights were
        # rotated with block 128 = head_dim along K, so their GEMV takes these codes as they are
        if self.tiled:
            # attention and the O projection as one call (for one token the projection's GEMV quantizes the merged row)
            check(lib.mi_gqa_decode_attn_tiled_linear_f32(self.q.ptr, self.kq.ptr, self.ks.ptr, self.vq.ptr, self.vs.ptr,
                                                          p(self.att), self.wo[0].ptr, self.wo[1].ptr, self.ao.ptr, B, Hq,
                                                          Hkv, D, self.T_cap, seq_len.ptr, t_max, H, self.att_ws.ptr,
                                                          self.att_ws.nbytes, s), "mi_gqa_decode_attn_tiled_linear_f32")
        else:
            check(lib.mi_gqa_decode_attn_cache_quant_i8(self.q.ptr, self.kq.ptr, self.ks.ptr, self.vq.ptr, self.vs.ptr,
                                                        p(self.att), self.ca.ptr, self.sa.ptr, B, Hq, Hkv, D, self.T_cap,
                                                        seq_len.ptr, t_max, self.att_ws.ptr, self.att_ws.nbytes, s),
                  "mi_gqa_decode_attn_cache_quant_i8")
            gemm_dequant(self.ca, self.sa, self.wo[0], self.wo[1], self.ao, s)
        if self.moe is None:
            check(lib.mi_rmsnorm_linear_f32(self.ao.ptr, xin.ptr, self.g2.ptr, self.eps, self.h1.ptr, p(self.hn),
                                            self.wgu[0].ptr, self.wgu[1].ptr, self.gu.ptr, B, 2 * I, H, self.block,
                                            self.lin_ws.ptr, self.lin_ws.nbytes, s), "mi_rmsnorm_linear_f32")
            check(lib.mi_swiglu_quant_f32_i8(self.gu.ptr, p(self.act), self.ci.ptr, self.si.ptr, B, I, self.block, s),
                  "mi_swiglu_quant_f32_i8")
            gemm_dequant(self.ci, self.si, self.wd[0], self.wd[1], self.dn, s)
        else:
            m = self.moe
            check(lib.mi_rmsnorm_f32(self.ao.ptr, xin.ptr, self.g2.ptr, self.eps, self.h1.ptr, self.hn.ptr, B, H, s),
                  "mi_rmsnorm_f32")
            moe_layer(self.hn, m["wr"], m["wg"], m["sg"], m["wu"], m["su"], m["wd"], m["sd"], self.dn, m["topk"],
                      self.moe_ws, stream=s)
        if out is not None:
            check(lib.mi_add_f32(self.h1.ptr, self.dn.ptr, out.ptr, B * H, s), "mi_add_f32")

    # the cache as row-major arrays [B,Hkv,T_cap,128] / [B,Hkv,T_cap], whatever layout the layer keeps it in
    def set_cache_rows(self, kq, ks, vq, vs):
        if self.tiled:
            kq, vq = kv_rows_to_tiled(kq, vq, self.T_cap)
        for buf, a in ((self.kq, kq), (self.ks, ks), (self.vq, vq), (self.vs, vs)):
            a = np.ascontiguousarray(a)
            check(lib.mi_memcpy_h2d(buf.ptr, a.ctypes.data, a.nbytes, None), "mi_memcpy_h2d")
        self.dev.sync()

    def get_cache_rows(self):
        kq, ks, vq, vs = (self.dev.download(b) for b in (self.kq, self.ks, self.vq, self.vs))
        if self.tiled:
            kq, vq = kv_tiled_to_rows(kq, vq)
        return kq, ks, vq, vs

    def fill_cache_from_rows(self, src, T, stream=None):
        """rotate + quantize fp32 rows [B*Hkv*T, 128] (device) into both halves of the cache (bench set-up)"""
        B, Hkv, D = self.B, self.Hkv, 128
        if not self.tiled:
            check(lib.mi_fwht_quant_f32_i8(src.ptr, self.kq.ptr, self.ks.ptr, B * Hkv * T, D, D, stream))
            check(lib.mi_fwht_quant_f32_i8(src.ptr, self.vq.ptr, self.vs.ptr, B * Hkv * T, D, D, stream))
            return
        mark = self.dev.mark()
        rows = self.dev.empty((B * Hkv * T, D), np.int8)
        check(lib.mi_fwht_quant_f32_i8(src.ptr, rows.ptr, self.ks.ptr, B * Hkv * T, D, D, stream))
        check(lib.mi_memcpy_d2d(self.vs.ptr, self.ks.ptr, B * Hkv * T * 4, stream))
        check(lib.mi_kv_tiled_from_rows_i8(rows.ptr, rows.ptr, self.kq.ptr, self.vq.ptr, B * Hkv, T, T, self.T_cap, stream))
        self.dev.sync(stream)
        self.dev.reset_to(mark)
