"""ctypes view of libllava_host.so: the C++ host classes (ggml_file, llava_context, llava_session) through the
flat C functions of host/capi.cpp.  One Python class per C++ class, one method per C++ method."""
import ctypes as C
import os

import numpy as np

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
_lib = None

RC_OK, RC_NOK, RC_NOT_TRACING = 0, 1, 5


def lib():
    global _lib
    if _lib is None:
        hip_path = os.path.join(PKG_DIR, "libllava_hip.so")
        path = os.path.join(PKG_DIR, "libllava_host.so")
        for p in (hip_path, path):
            if not os.path.exists(p):
                raise FileNotFoundError(f"{p} is not built; run python llama-vulkan_amd/build.py")
        C.CDLL(hip_path, mode=C.RTLD_GLOBAL)
        L = C.CDLL(path)
        vp, u, cp = C.c_void_p, C.c_uint, C.c_char_p
        sig = {
            "llh_file_open": (vp, [cp]), "llh_file_close": (None, [vp]), "llh_file_is_open": (C.c_int, [vp]),
            "llh_file_error": (u, [vp, cp, u]), "llh_file_header": (None, [vp, C.POINTER(u)]), "llh_file_print_info": (None, [vp]),
            "llh_file_tensor_at": (u, [vp, u, cp, u, C.POINTER(u), C.POINTER(C.c_ulonglong), C.POINTER(u), C.POINTER(u), C.POINTER(C.c_ulonglong)]),
            "llh_file_tensor": (C.c_int, [vp, cp, C.POINTER(u), C.POINTER(C.c_ulonglong), C.POINTER(u), C.POINTER(u), C.POINTER(C.c_ulonglong)]),
            "llh_file_token": (u, [vp, u, cp, u, C.POINTER(C.c_float)]),
            "llh_file_tokenize": (u, [vp, cp, u, C.c_int, C.POINTER(u), u]), "llh_file_detokenize": (u, [vp, C.POINTER(u), u, cp, u]),
            "llh_context_new": (vp, []), "llh_context_free": (None, [vp]), "llh_context_load": (C.c_int, [vp, cp, C.c_int]),
            "llh_context_error": (u, [vp, cp, u]), "llh_context_run": (C.c_int, [vp, C.c_int, C.POINTER(cp)]),
            "llh_context_open_file": (C.c_int, [vp, cp]),
            "llh_server_start": (vp, [vp, C.c_ushort, cp]), "llh_server_port": (u, [vp]), "llh_server_stop": (None, [vp]),
            "llh_session_new": (vp, [vp]), "llh_session_free": (None, [vp]), "llh_session_good": (C.c_int, [vp]),
            "llh_session_set_text": (C.c_int, [vp, cp, u]), "llh_session_add_text": (C.c_int, [vp, cp, u]),
            "llh_session_push_token": (C.c_int, [vp, u]), "llh_session_token_count": (u, [vp]), "llh_session_tokens": (u, [vp, C.POINTER(u), u]),
            "llh_session_start": (C.c_int, [vp]), "llh_session_finish": (u, [vp, C.c_int]), "llh_session_predict": (u, [vp, C.c_int]),
            "llh_session_rewind": (None, [vp, u]), "llh_session_set_options": (u, [vp, u]), "llh_session_is_tracing": (C.c_int, [vp]),
            "llh_session_save_frame": (u, [vp, cp]), "llh_session_snapshot": (u, [vp, cp]), "llh_session_restore": (u, [vp, cp]),
            "llh_session_seed": (None, [vp, u]), "llh_session_backlog": (u, [vp]), "llh_session_device": (vp, [vp]),
            "llh_sample_token": (u, [C.POINTER(C.c_float), u, C.POINTER(u), u, C.POINTER(C.c_float), u, C.POINTER(u), C.POINTER(C.c_float), u,
                                     C.POINTER(u), C.POINTER(C.c_float), C.POINTER(C.c_int)]), "llh_session_tokens_in_gpu": (u, [vp]),
            "llh_session_logits": (u, [vp, C.c_void_p, u]), "llh_session_spevars": (None, [vp, C.POINTER(u)]), "llh_session_layer_count": (u, [vp]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def _text(fn, handle, cap=4096):
    buf = C.create_string_buffer(cap)
    n = fn(handle, buf, cap)
    return buf.raw[:min(n, cap)].decode(errors="replace")


class GgmlFile:
    """ggml_file"""

    def __init__(self, path):
        self.h = lib().llh_file_open(os.fsencode(path))

    def close(self):
        if self.h:
            lib().llh_file_close(self.h)
            self.h = None

    def is_open(self):
        return bool(lib().llh_file_is_open(self.h))

    def error(self):
        return _text(lib().llh_file_error, self.h)

    def header(self):
        out = (C.c_uint * 10)()
        lib().llh_file_header(self.h, out)
        keys = ["file_version", "vocab", "dim", "multiple_of", "heads", "layers", "rot", "ftype", "ff", "n_tensors"]
        return dict(zip(keys, [int(v) for v in out]))

    def tensors(self):
        out = []
        name = C.create_string_buffer(256)
        for i in range(self.header()["n_tensors"]):
            ft, off, s1, s2, size = C.c_uint(), C.c_ulonglong(), C.c_uint(), C.c_uint(), C.c_ulonglong()
            n = lib().llh_file_tensor_at(self.h, i, name, 256, C.byref(ft), C.byref(off), C.byref(s1), C.byref(s2), C.byref(size))
            out.append(dict(name=name.raw[:n].decode(), ftype=ft.value, offset=off.value, rows=s1.value, cols=s2.value, size=size.value))
        return out

    def tensor(self, name):
        ft, off, s1, s2, size = C.c_uint(), C.c_ulonglong(), C.c_uint(), C.c_uint(), C.c_ulonglong()
        if lib().llh_file_tensor(self.h, name.encode(), C.byref(ft), C.byref(off), C.byref(s1), C.byref(s2), C.byref(size)):
            raise KeyError(name)
        return dict(ftype=ft.value, offset=off.value, rows=s1.value, cols=s2.value, size=size.value)

    def token(self, i):
        buf = C.create_string_buffer(256)
        score = C.c_float()
        n = lib().llh_file_token(self.h, i, buf, 256, C.byref(score))
        return buf.raw[:n], score.value

    def tokenize(self, text: bytes, bos: bool):
        cap = 4 * len(text) + 8
        out = (C.c_uint * cap)()
        n = lib().llh_file_tokenize(self.h, text, len(text), int(bos), out, cap)
        return [int(out[i]) for i in range(n)]

    def detokenize(self, ids):
        arr = (C.c_uint * max(len(ids), 1))(*ids)
        cap = 64 * len(ids) + 8
        buf = C.create_string_buffer(cap)
        n = lib().llh_file_detokenize(self.h, arr, len(ids), buf, cap)
        return buf.raw[:n]


def sample_token(logits, history, mu, seed):
    """llava_session::sample_token (the stochastic pick of llava_session.cpp:154-194) on given logits and token history.
    Returns (token, new mu, kept ids, kept probabilities, their sum, index drawn among the kept)."""
    n = len(logits)
    lg = (C.c_float * n)(*[float(v) for v in logits])
    hist = (C.c_uint * max(len(history), 1))(*[int(t) for t in history])
    mu_io, ids, ps = C.c_float(mu), (C.c_uint * n)(), (C.c_float * n)()
    count, total, pick = C.c_uint(), C.c_float(), C.c_int()
    tok = lib().llh_sample_token(lg, n, hist, len(history), C.byref(mu_io), seed, ids, ps, n, C.byref(count), C.byref(total), C.byref(pick))
    k = count.value
    return tok, mu_io.value, [int(ids[i]) for i in range(k)], [float(ps[i]) for i in range(k)], total.value, pick.value


class LlavaContext:
    """llava_context"""

    def __init__(self):
        self.h = lib().llh_context_new()

    def load_model(self, path, device=0):
        return lib().llh_context_load(self.h, os.fsencode(path), device) == 0

    def open_model_file(self, path):
        """parse only: vocabulary and tensor table, no device"""
        return lib().llh_context_open_file(self.h, os.fsencode(path)) == 0

    def error(self):
        return _text(lib().llh_context_error, self.h)

    def close(self):
        if self.h:
            lib().llh_context_free(self.h)
            self.h = None


class LlavaServer:
    """lsrv::llava_server running its poll loop on a thread of its own; port 0 takes a free port"""

    def __init__(self, ctx, port=0, bind_address="127.0.0.1"):
        self.h = lib().llh_server_start(ctx.h, port, bind_address.encode())
        if not self.h:
            raise OSError("the server socket could not be opened")
        self.port = lib().llh_server_port(self.h)

    def stop(self):
        """kills the sessions, waits for their threads, closes the connections"""
        if self.h:
            lib().llh_server_stop(self.h)
            self.h = None


class LlavaSession:
    """llava_session"""

    def __init__(self, ctx):
        self.ctx = ctx
        self.h = lib().llh_session_new(ctx.h)

    def close(self):
        if self.h:
            lib().llh_session_free(self.h)
            self.h = None

    def good(self):
        return bool(lib().llh_session_good(self.h))

    def set_text(self, text: bytes):
        return bool(lib().llh_session_set_text(self.h, text, len(text)))

    def add_text(self, text: bytes):
        return bool(lib().llh_session_add_text(self.h, text, len(text)))

    def push_token(self, t):
        return bool(lib().llh_session_push_token(self.h, int(t)))

    def token_count(self):
        return lib().llh_session_token_count(self.h)

    def tokens(self):
        n = self.token_count()
        out = (C.c_uint * max(n, 1))()
        lib().llh_session_tokens(self.h, out, n)
        return [int(out[i]) for i in range(n)]

    def start(self):
        return bool(lib().llh_session_start(self.h))

    def finish(self, deterministic=False):
        return lib().llh_session_finish(self.h, int(deterministic))

    def predict(self, deterministic=False):
        return lib().llh_session_predict(self.h, int(deterministic))

    def rewind(self, n):
        lib().llh_session_rewind(self.h, n)

    def device_session(self):
        """the lv_session handle (an integer address) behind this object"""
        return lib().llh_session_device(self.h)

    def set_options(self, o):
        return lib().llh_session_set_options(self.h, o)

    def is_tracing(self):
        return bool(lib().llh_session_is_tracing(self.h))

    def save_frame(self, path):
        return lib().llh_session_save_frame(self.h, os.fsencode(path))

    def snapshot(self, path):
        return lib().llh_session_snapshot(self.h, os.fsencode(path))

    def restore(self, path):
        return lib().llh_session_restore(self.h, os.fsencode(path))

    def seed(self, s):
        lib().llh_session_seed(self.h, s)

    def backlog(self):
        return lib().llh_session_backlog(self.h)

    def tokens_in_gpu(self):
        return lib().llh_session_tokens_in_gpu(self.h)

    def logits(self):
        n = lib().llh_session_logits(self.h, None, 0)
        out = np.empty(n, dtype=np.float32)
        lib().llh_session_logits(self.h, out.ctypes.data_as(C.c_void_p), n)
        return out

    def spevars(self):
        out = (C.c_uint * 21)()
        lib().llh_session_spevars(self.h, out)
        keys = ["head_count", "quarterrot", "backlog", "max_wgs", "max_wgs_bits", "ff_size", "softmax_head_per_wavefront", "backlog_bits",
                "rot_bits", "rot", "matmul_dim_row_per_wavefront", "matmul_dim_row_worker_count", "matmul_dim_row_worker_count_log2",
                "matmul_dim_q4_block_count_per_worker", "matmul_dim_q4_blocks_per_row", "matmul_ff_row_per_wavefront",
                "matmul_ff_row_worker_count", "matmul_ff_row_worker_count_log2", "matmul_ff_q4_block_count_per_worker",
                "matmul_ff_q4_blocks_per_row", "batch_enabled"]
        return dict(zip(keys, [int(v) for v in out]))

    def layer_count(self):
        return lib().llh_session_layer_count(self.h)
