"""MI355X-native decode path behind the llama-vulkan C++ surface: Python view of the native libraries.

The directory name contains a hyphen, so import it with
``importlib.import_module("llama-vulkan_amd")``.

This module only binds what is built in-tree with ctypes:

* ``hip()``    -> libllava_hip.so, the gfx950 C-ABI declared in include/llava_hip.h
* ``host()``   -> libllava_host.so, the C++ host classes (ggml_file, llava_session) through their C shim
* ``mkggml()`` -> libmkggml.so, the deterministic synthetic GGJT writer

There is no fallback: a missing library raises, it is never replaced by a CPU path.
"""
import ctypes as C
import os

import numpy as np

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT_DIR = os.path.dirname(PKG_DIR)

LV_F32, LV_F16, LV_Q4_0, LV_Q8_0 = 0, 1, 2, 8
PATH_AUTO, PATH_KERNELS, PATH_GRAPH, PATH_PERSISTENT = range(4)
TRACE_NORM_IN, TRACE_POST_ATTN, TRACE_POST_ATTN_NORM, TRACE_FF, TRACE_OUT, TRACE_ATTN = range(6)


class LvError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"lv status {code}: {text}")
        self.code = code


class TensorDesc(C.Structure):
    _fields_ = [("name", C.c_char_p), ("ftype", C.c_uint32), ("offset", C.c_uint64), ("rows", C.c_uint32),
                ("cols", C.c_uint32), ("size", C.c_uint64)]


class HParams(C.Structure):
    _fields_ = [("file_version", C.c_uint32), ("vocab", C.c_uint32), ("dim", C.c_uint32), ("heads", C.c_uint32),
                ("layers", C.c_uint32), ("rot", C.c_uint32), ("ff", C.c_uint32)]


class MkgConfig(C.Structure):
    _fields_ = [("vocab", C.c_uint32), ("dim", C.c_uint32), ("heads", C.c_uint32), ("layers", C.c_uint32),
                ("ff", C.c_uint32), ("multiple_of", C.c_uint32), ("wtype", C.c_uint32), ("seed", C.c_uint64),
                ("sigma", C.c_float), ("tok_type", C.c_uint32)]


_libs = {}


def _load(name):
    if name not in _libs:
        path = os.path.join(PKG_DIR, name)
        if not os.path.exists(path):
            raise FileNotFoundError(
                f"{path} is not built; run `python -c \"import __graft_entry__ as g; g.build()\"` "
                f"(or python llama-vulkan_amd/build.py)")
        _libs[name] = C.CDLL(path, mode=C.RTLD_GLOBAL)
    return _libs[name]


def exported_symbols():
    """Names include/llava_hip.h declares (parsed from the header, used by the symbol-presence test)."""
    import re
    text = open(os.path.join(ROOT_DIR, "include", "llava_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lv_[a-z0-9_]+)\s*\(", text)))


# ----------------------------------------------------------------------------------------------------------
# libllava_hip.so
# ----------------------------------------------------------------------------------------------------------
_VP, _U32, _U64, _I = C.c_void_p, C.c_uint32, C.c_uint64, C.c_int
_HIP_SIGS = {
    "lv_ctx_create": [_I, C.POINTER(_VP)],
    "lv_ctx_destroy": [_VP],
    "lv_ctx_info": [_VP, C.c_char_p, C.c_size_t, C.POINTER(_U32), C.POINTER(_U64)],
    "lv_ctx_sync": [_VP],
    "lv_ctx_timer_start": [_VP],
    "lv_ctx_timer_stop": [_VP, C.POINTER(C.c_float)],
    "lv_session_timer_start": [_VP],
    "lv_session_timer_stop": [_VP, C.POINTER(C.c_float)],
    "lv_model_upload": [_VP, _VP, _U64, C.POINTER(HParams), C.POINTER(TensorDesc), _U32, C.POINTER(_VP)],
    "lv_model_destroy": [_VP],
    "lv_model_hparams": [_VP, C.POINTER(HParams)],
    "lv_model_arena_bytes": [_VP, C.POINTER(_U64)],
    "lv_session_create": [_VP, C.POINTER(_VP)],
    "lv_session_destroy": [_VP],
    "lv_session_reserve": [_VP, _U32],
    "lv_session_backlog": [_VP, C.POINTER(_U32)],
    "lv_session_use_graph": [_VP, _I],
    "lv_session_set_path": [_VP, _I],
    "lv_session_set_wait_limit": [_VP, C.c_uint32],
    "lv_session_set_xcd_handover": [_VP, _I],
    "lv_session_xcd_handover": [_VP, C.POINTER(_I)],
    "lv_session_path": [_VP, C.POINTER(_I)],
    "lv_step_begin": [_VP, _VP, _U32, _U32],
    "lv_step_wait": [_VP],
    "lv_logits_read": [_VP, _VP],
    "lv_session_set_all_logits": [_VP, _I],
    "lv_logits_read_rows": [_VP, _U32, _U32, _VP],
    "lv_argmax": [_VP, C.POINTER(_U32)],
    "lv_kv_read": [_VP, _U32, _I, _U32, _VP],
    "lv_kv_write": [_VP, _U32, _I, _U32, _VP],
    "lv_trace_enable": [_VP, _I],
    "lv_trace_read": [_VP, _U32, _I, _VP, _U32],
    "lv_trace_rows": [_VP, C.POINTER(_U32)],
    "lv_trace_read_rows": [_VP, _U32, _I, _U32, _U32, _VP],
    "lv_dev_alloc": [_VP, _U64, C.POINTER(_VP)],
    "lv_dev_free": [_VP, _VP],
    "lv_dev_upload": [_VP, _VP, _VP, _U64],
    "lv_dev_download": [_VP, _VP, _VP, _U64],
    "lv_dev_zero": [_VP, _VP, _U64],
    "lv_dev_copy": [_VP, _VP, _VP, _U64],
    "lv_dev_read": [_VP, _VP, _U64],
    "lv_matrix_upload": [_VP, _VP, _U32, _U32, _U32, _U32, C.POINTER(_VP)],
    "lv_matrix_destroy": [_VP],
    "lv_matrix_bytes": [_VP, C.POINTER(_U64)],
    "lv_kernel_dequant": [_VP, _VP, _U32, _U32, _VP],
    "lv_kernel_gemv": [_VP, _VP, _VP, _VP, _U32, _I],
    "lv_kernel_gemm": [_VP, _VP, _VP, _VP, _U32, _I],
    "lv_kernel_gemv_silu": [_VP, _VP, _VP, _VP, _VP, _U32],
    "lv_kernel_normalize": [_VP, _VP, _VP, _VP, _U32, _U32],
    "lv_kernel_kv_append": [_VP, _VP, _VP, _U32, _U32, _U32, _U32],
    "lv_kernel_attention": [_VP, _VP, _VP, _VP, _VP, _U32, _U32, _U32, _U32, _U32],
    "lv_kernel_attention_static": [_VP, _VP, _VP, _VP, _VP, _U32, _U32, _U32, _U32, _U32],
}


def hip():
    lib = _load("libllava_hip.so")
    if not getattr(lib, "_lv_bound", False):
        for name, args in _HIP_SIGS.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = C.c_int
        lib.lv_last_error.restype = C.c_char_p
        lib.lv_last_error.argtypes = []
        lib._lv_bound = True
    return lib


def check(rc):
    if rc != 0:
        raise LvError(rc, hip().lv_last_error().decode(errors="replace"))


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


class Context:
    """lv_ctx plus small numpy conveniences for device buffers."""

    def __init__(self, device=0):
        self.lib = hip()
        self.h = C.c_void_p()
        check(self.lib.lv_ctx_create(device, C.byref(self.h)))

    def close(self):
        if self.h:
            self.lib.lv_ctx_destroy(self.h)
            self.h = C.c_void_p()

    def info(self):
        name = C.create_string_buffer(256)
        cus, hbm = C.c_uint32(), C.c_uint64()
        check(self.lib.lv_ctx_info(self.h, name, 256, C.byref(cus), C.byref(hbm)))
        return name.value.decode(), cus.value, hbm.value

    def sync(self):
        check(self.lib.lv_ctx_sync(self.h))

    def timer_start(self):
        check(self.lib.lv_ctx_timer_start(self.h))

    def timer_stop(self):
        ms = C.c_float()
        check(self.lib.lv_ctx_timer_stop(self.h, C.byref(ms)))
        return ms.value

    def alloc(self, nbytes):
        p = C.c_void_p()
        check(self.lib.lv_dev_alloc(self.h, nbytes, C.byref(p)))
        return p

    def free(self, p):
        check(self.lib.lv_dev_free(self.h, p))

    def to_device(self, arr):
        arr = np.ascontiguousarray(arr)
        p = self.alloc(max(arr.nbytes, 4))
        check(self.lib.lv_dev_upload(self.h, p, _ptr(arr), arr.nbytes))
        return p

    def zeros(self, nbytes):
        p = self.alloc(nbytes)
        check(self.lib.lv_dev_zero(self.h, p, nbytes))
        self.sync()
        return p

    def to_host(self, p, shape, dtype):
        out = np.empty(shape, dtype=dtype)
        check(self.lib.lv_dev_download(self.h, _ptr(out), p, out.nbytes))
        return out

    def matrix(self, blocks, ftype, rows, cols, file_version=3):
        blocks = np.ascontiguousarray(blocks)
        m = C.c_void_p()
        check(self.lib.lv_matrix_upload(self.h, _ptr(blocks), ftype, file_version, rows, cols, C.byref(m)))
        return m

    def matrix_free(self, m):
        check(self.lib.lv_matrix_destroy(m))


# ----------------------------------------------------------------------------------------------------------
# libmkggml.so
# ----------------------------------------------------------------------------------------------------------
def mkggml():
    lib = _load("libmkggml.so")
    if not getattr(lib, "_bound", False):
        lib.mkg_write_model.argtypes = [C.c_char_p, C.POINTER(MkgConfig)]
        lib.mkg_write_model.restype = C.c_int
        lib.mkg_quant_bytes.argtypes = [C.c_uint32, C.c_uint64, C.c_uint64]
        lib.mkg_quant_bytes.restype = C.c_size_t
        lib.mkg_fill_quant.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint64, C.c_float]
        lib.mkg_fill_quant.restype = None
        lib.mkg_fill_normal.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint64, C.c_uint64, C.c_float]
        lib.mkg_fill_normal.restype = None
        lib.mkg_fill_tokens.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint64]
        lib.mkg_fill_tokens.restype = None
        lib._bound = True
    return lib


PRESETS = {
    "7b": dict(vocab=32000, dim=4096, heads=32, layers=32, ff=11008),
    "13b": dict(vocab=32000, dim=5120, heads=40, layers=40, ff=13824),
    "tiny": dict(vocab=512, dim=256, heads=4, layers=2, ff=704),
}


def write_model(path, wtype=LV_Q4_0, seed=0, sigma=0.02, preset=None, tok_type=0, **shape):
    """tok_type: 0 = f32 embedding table (the published configs), LV_Q4_0 / LV_Q8_0 = quantised like the matrices"""
    cfg = dict(PRESETS[preset]) if preset else {}
    cfg.update(shape)
    c = MkgConfig(cfg["vocab"], cfg["dim"], cfg["heads"], cfg["layers"], cfg["ff"], 256, wtype, seed, sigma, tok_type)
    rc = mkggml().mkg_write_model(os.fsencode(path), C.byref(c))
    if rc != 0:
        raise OSError(-rc, os.strerror(-rc), path)
    return path


def synth_quant(wtype, rows, cols, seed, tensor_id=0, sigma=0.02):
    """rows x cols quantised matrix as raw GGML blocks (uint8 array)."""
    lib = mkggml()
    buf = np.empty(lib.mkg_quant_bytes(wtype, rows, cols), dtype=np.uint8)
    lib.mkg_fill_quant(_ptr(buf), wtype, rows, cols, seed, tensor_id, sigma)
    return buf


def synth_normal(rows, cols, seed, tensor_id=0, sigma=1.0):
    out = np.empty((rows, cols), dtype=np.float32)
    mkggml().mkg_fill_normal(_ptr(out), rows, cols, seed, tensor_id, sigma)
    return out


def synth_tokens(n, lo, hi, seed):
    out = np.empty(n, dtype=np.uint32)
    mkggml().mkg_fill_tokens(_ptr(out), n, lo, hi, seed)
    return out


# ----------------------------------------------------------------------------------------------------------
# GGJT table reader for Python callers of the C-ABI (the C++ ggml_file class is the product parser; this is
# the same 40 lines of format knowledge for scripts that hand lv_model_upload a table)
# ----------------------------------------------------------------------------------------------------------
def _tensor_bytes(ftype, n, file_version=3):
    """file version 1 stores fp32 block scales, later versions fp16 ones (reference: ggml_file.cpp:95-122)"""
    wide = 2 if file_version == 1 else 0
    return {LV_F32: n * 4, LV_F16: n * 2, LV_Q4_0: n // 32 * (18 + wide), LV_Q8_0: n // 32 * (34 + wide)}[ftype]


def read_ggjt_table(path):
    """Returns (mmap-backed uint8 array, header dict, [(name, ftype, offset, rows, cols, size)])."""
    data = np.memmap(path, dtype=np.uint8, mode="r")
    hdr = np.frombuffer(data[:36], dtype=np.uint32)
    if hdr[0] != 0x67676A74:
        raise ValueError("not a GGJT file")
    keys = ["magic", "file_version", "vocab", "dim", "multiple_of", "heads", "layers", "rot", "ftype"]
    header = {k: int(v) for k, v in zip(keys, hdr)}
    cur = 36
    for _ in range(header["vocab"]):
        ln = int(np.frombuffer(data[cur:cur + 4], dtype=np.uint32)[0])
        cur += 4 + ln + 4
    table = []
    total = data.shape[0]
    while cur != total:
        n_dims, name_len, ftype = (int(v) for v in np.frombuffer(data[cur:cur + 12], dtype=np.uint32))
        cur += 12
        ne = [int(v) for v in np.frombuffer(data[cur:cur + 4 * n_dims], dtype=np.uint32)]
        cur += 4 * n_dims
        name = bytes(data[cur:cur + name_len]).decode()
        cur += name_len
        rows, cols = (ne[1], ne[0]) if n_dims == 2 else (ne[0], 1)
        offset = (cur + 31) & ~31
        size = _tensor_bytes(ftype, rows * cols, header["file_version"])
        table.append((name, ftype, offset, rows, cols, size))
        cur = offset + size
    for name, _, _, rows, _, _ in table:
        if name.startswith("layers.0.feed_forward.w1"):
            header["ff"] = rows
    return data, header, table


class Model:
    """A GGJT file uploaded through lv_model_upload."""

    def __init__(self, ctx, path):
        self.ctx = ctx
        self.lib = ctx.lib
        data, header, table = read_ggjt_table(path)
        self.header = header
        descs = (TensorDesc * len(table))()
        self._names = [t[0].encode() for t in table]
        for d, t, nm in zip(descs, table, self._names):
            d.name, d.ftype, d.offset, d.rows, d.cols, d.size = nm, t[1], t[2], t[3], t[4], t[5]
        hp = HParams(header["file_version"], header["vocab"], header["dim"], header["heads"], header["layers"],
                     header["rot"], header["ff"])
        self.h = C.c_void_p()
        check(self.lib.lv_model_upload(ctx.h, C.c_void_p(data.ctypes.data), data.shape[0], C.byref(hp), descs,
                                       len(table), C.byref(self.h)))
        del data

    def close(self):
        if self.h:
            self.lib.lv_model_destroy(self.h)
            self.h = C.c_void_p()


class Session:
    """lv_session: one stream, one K/V cache, one captured decode graph."""

    def __init__(self, model, backlog=128):
        self.model = model
        self.lib = model.lib
        self.h = C.c_void_p()
        check(self.lib.lv_session_create(model.h, C.byref(self.h)))
        self.reserve(backlog)

    def close(self):
        if self.h:
            self.lib.lv_session_destroy(self.h)
            self.h = C.c_void_p()

    def reserve(self, backlog):
        check(self.lib.lv_session_reserve(self.h, backlog))

    def use_graph(self, on):
        check(self.lib.lv_session_use_graph(self.h, int(on)))

    def set_path(self, path):
        check(self.lib.lv_session_set_path(self.h, int(path)))

    def set_wait_limit(self, polls):
        check(self.lib.lv_session_set_wait_limit(self.h, int(polls)))

    def set_xcd_handover(self, on):
        check(self.lib.lv_session_set_xcd_handover(self.h, int(on)))

    def xcd_handover(self):
        """did the last persistent step keep the hand-overs inside a head inside one XCD?"""
        used = C.c_int()
        check(self.lib.lv_session_xcd_handover(self.h, C.byref(used)))
        return bool(used.value)

    def path(self):
        p = C.c_int()
        check(self.lib.lv_session_path(self.h, C.byref(p)))
        return p.value

    def begin(self, tokens, pos):
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        check(self.lib.lv_step_begin(self.h, _ptr(t), t.shape[0], pos))

    def wait(self):
        check(self.lib.lv_step_wait(self.h))

    def timer_start(self):
        check(self.lib.lv_session_timer_start(self.h))

    def timer_stop(self):
        ms = C.c_float()
        check(self.lib.lv_session_timer_stop(self.h, C.byref(ms)))
        return ms.value

    def logits(self):
        out = np.empty(self.model.header["vocab"], dtype=np.float32)
        check(self.lib.lv_logits_read(self.h, _ptr(out)))
        return out

    def keep_all_logits(self, on=True):
        check(self.lib.lv_session_set_all_logits(self.h, int(on)))

    def logits_rows(self, row0, n_rows):
        """logits of rows row0 .. row0 + n_rows - 1 of the last step (needs keep_all_logits before that step)"""
        out = np.empty((n_rows, self.model.header["vocab"]), dtype=np.float32)
        check(self.lib.lv_logits_read_rows(self.h, row0, n_rows, _ptr(out)))
        return out

    def argmax(self):
        t = C.c_uint32()
        check(self.lib.lv_argmax(self.h, C.byref(t)))
        return t.value

    def kv(self, layer, which, n_tokens):
        out = np.empty((n_tokens, self.model.header["dim"]), dtype=np.uint16)
        check(self.lib.lv_kv_read(self.h, layer, which, n_tokens, _ptr(out)))
        return out

    def kv_write(self, layer, which, rows):
        rows = np.ascontiguousarray(rows, dtype=np.uint16)
        check(self.lib.lv_kv_write(self.h, layer, which, rows.shape[0], _ptr(rows)))

    def trace_enable(self, on=True):
        check(self.lib.lv_trace_enable(self.h, int(on)))

    def trace(self, layer, which):
        n = self.model.header["ff"] if which == TRACE_FF else self.model.header["dim"]
        if which == TRACE_ATTN:
            rows = C.c_uint32()
            check(self.lib.lv_session_backlog(self.h, C.byref(rows)))
            n = rows.value * self.model.header["heads"]
        out = np.empty(n, dtype=np.float32)
        check(self.lib.lv_trace_read(self.h, layer, which, _ptr(out), n))
        return out

    def trace_rows(self):
        """rows the last recorded step left in the trace buffers"""
        rows = C.c_uint32()
        check(self.lib.lv_trace_rows(self.h, C.byref(rows)))
        return rows.value

    def trace_all(self, layer, which, row0=0, n_rows=None):
        """rows [row0, row0 + n_rows) of one trace buffer of the last recorded step, shape (n_rows, floats per row)"""
        n = self.model.header["ff"] if which == TRACE_FF else self.model.header["dim"]
        if which == TRACE_ATTN:
            rows = C.c_uint32()
            check(self.lib.lv_session_backlog(self.h, C.byref(rows)))
            n = rows.value * self.model.header["heads"]
        if n_rows is None:
            n_rows = self.trace_rows() - row0
        out = np.empty((n_rows, n), dtype=np.float32)
        check(self.lib.lv_trace_read_rows(self.h, layer, which, row0, n_rows, _ptr(out)))
        return out
