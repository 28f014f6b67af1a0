"""ctypes view of the CPU checker (liboracle.so) and of the reference-built parser (_ref/libref_ggml.so).

TEST INFRASTRUCTURE ONLY.  Imported by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline
leg, as the checker; the product never routes through it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboracle.so")
REF_PATH = os.path.join(HERE, "_ref", "libref_ggml.so")

F32, F16, Q4_0, Q8_0 = 0, 1, 2, 8
TR_NORM_IN, TR_POST_ATTN, TR_POST_ATTN_NORM, TR_FF, TR_OUT, TR_ATTN = range(6)


class HParams(C.Structure):
    _fields_ = [(k, C.c_uint32) for k in
                ("file_version", "vocab", "dim", "multiple_of", "heads", "layers", "rot", "ftype", "ff", "n_tensors")]


_lib = None


def build():
    subprocess.run(["make", "-C", HERE, "all"], check=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        vp, u32, u64, f32p = C.c_void_p, C.c_uint32, C.c_uint64, C.c_void_p
        L.orc_half_to_float.argtypes = [C.c_uint16]
        L.orc_half_to_float.restype = C.c_float
        L.orc_float_to_half.argtypes = [C.c_float]
        L.orc_float_to_half.restype = C.c_uint16
        L.orc_tensor_bytes.argtypes = [u32, u32, u64]
        L.orc_tensor_bytes.restype = C.c_size_t
        L.orc_dequant.argtypes = [vp, u32, u32, f32p, u32]
        L.orc_gemv.argtypes = [f32p, vp, u32, u32, u32, u32, f32p, u32, C.c_int, u32]
        L.orc_gemv_silu.argtypes = [f32p, vp, vp, u32, u32, u32, u32, f32p, u32, u32]
        L.orc_normalize.argtypes = [f32p, f32p, f32p, u32, u32, u32]
        L.orc_normalize.restype = None
        L.orc_kv_append.argtypes = [vp, f32p, u32, u32, u32]
        L.orc_kv_append.restype = None
        L.orc_mhsa.argtypes = [f32p, vp, f32p, u32, u32, u32, u32, u32]
        L.orc_mhsa.restype = None
        L.orc_softmax.argtypes = [f32p, u32, u32, u32, u32, u32]
        L.orc_softmax.restype = None
        L.orc_kqv.argtypes = [f32p, vp, f32p, u32, u32, u32, u32]
        L.orc_kqv.restype = None
        L.orc_sample_greedy.argtypes = [f32p, u32]
        L.orc_sample_greedy.restype = u32
        L.orc_model_open.argtypes = [C.c_char_p]
        L.orc_model_open.restype = vp
        L.orc_model_close.argtypes = [vp]
        L.orc_model_close.restype = None
        L.orc_model_hparams.argtypes = [vp, C.POINTER(HParams)]
        L.orc_model_hparams.restype = None
        L.orc_model_tensor.argtypes = [vp, C.c_char_p, C.POINTER(u32), C.POINTER(u64), C.POINTER(u32), C.POINTER(u32),
                                       C.POINTER(u64)]
        L.orc_model_data.argtypes = [vp, u64]
        L.orc_model_data.restype = vp
        L.orc_session_new.argtypes = [vp, u32]
        L.orc_session_new.restype = vp
        L.orc_session_free.argtypes = [vp]
        L.orc_session_free.restype = None
        L.orc_session_pos.argtypes = [vp]
        L.orc_session_pos.restype = u32
        L.orc_session_rewind.argtypes = [vp, u32]
        L.orc_session_rewind.restype = None
        L.orc_session_eval.argtypes = [vp, vp, u32, f32p, f32p]
        L.orc_session_kv.argtypes = [vp, u32, C.c_int]
        L.orc_session_kv.restype = vp
        L.orc_session_trace.argtypes = [vp, u32, C.c_int, C.POINTER(u32)]
        L.orc_session_trace.restype = vp
        L.orc_session_kv_load.argtypes = [vp, u32, C.c_int, vp, u32]
        L.orc_session_set_pos.argtypes = [vp, u32]
        L.orc_num_threads.argtypes = []
        L.orc_forward_f64.argtypes = [vp, vp, u32, u32, vp, vp, vp]
        L.orc_forward_f64_activation_bits.argtypes = [C.c_int]
        L.orc_forward_f64_activation_bits.restype = None
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def half_to_float(bits):
    L = lib()
    return np.array([L.orc_half_to_float(int(b)) for b in np.asarray(bits).ravel()], dtype=np.float32)


def float_to_half(vals):
    L = lib()
    return np.array([L.orc_float_to_half(float(v)) for v in np.asarray(vals, dtype=np.float32).ravel()], dtype=np.uint16)


def dequant(blocks, ftype, count, file_version=3):
    blocks = np.ascontiguousarray(blocks)
    out = np.empty(count, dtype=np.float32)
    rc = lib().orc_dequant(_p(blocks), ftype, file_version, _p(out), count)
    if rc:
        raise ValueError("orc_dequant refused the arguments")
    return out


def gemv(blocks, ftype, rows, cols, x, out=None, accumulate=False, workers=0, file_version=3):
    x = _f32(x).reshape(-1, cols)
    batch = x.shape[0]
    blocks = np.ascontiguousarray(blocks)
    if out is None:
        out = np.zeros((batch, rows), dtype=np.float32)
    else:
        out = _f32(out).reshape(batch, rows).copy()
    rc = lib().orc_gemv(_p(out), _p(blocks), ftype, file_version, rows, cols, _p(x), batch, int(accumulate), workers)
    if rc:
        raise ValueError("orc_gemv refused the arguments")
    return out


def gemv_silu(w3, w1, ftype, rows, cols, x, workers=0, file_version=3):
    x = _f32(x).reshape(-1, cols)
    batch = x.shape[0]
    w3, w1 = np.ascontiguousarray(w3), np.ascontiguousarray(w1)
    out = np.zeros((batch, rows), dtype=np.float32)
    rc = lib().orc_gemv_silu(_p(out), _p(w3), _p(w1), ftype, file_version, rows, cols, _p(x), batch, workers)
    if rc:
        raise ValueError("orc_gemv_silu refused the arguments")
    return out


def normalize(x, w, wgs=0):
    x = _f32(x)
    x2 = x.reshape(-1, x.shape[-1])
    w = _f32(w)
    out = np.empty_like(x2)
    lib().orc_normalize(_p(out), _p(x2), _p(w), x2.shape[1], x2.shape[0], wgs)
    return out.reshape(x.shape)


def kv_append(cache, rows, pos):
    """cache: uint16 [backlog][dim] (modified in place); rows: float32 [batch][dim]"""
    rows = _f32(rows).reshape(-1, cache.shape[1])
    lib().orc_kv_append(_p(cache), _p(rows), pos, cache.shape[1], rows.shape[0])
    return cache


def mhsa(kcache, q, pos, heads, rot):
    q = _f32(q).reshape(-1, heads * rot)
    backlog = kcache.shape[0]
    out = np.zeros((q.shape[0], backlog, heads), dtype=np.float32)
    lib().orc_mhsa(_p(out), _p(kcache), _p(q), pos, backlog, heads, rot, q.shape[0])
    return out


def softmax(scores, pos, rot):
    s = _f32(scores).copy()
    batch, backlog, heads = s.shape
    lib().orc_softmax(_p(s), pos, backlog, heads, rot, batch)
    return s


def kqv(vcache, attn, heads, rot):
    attn = _f32(attn)
    batch, backlog, _ = attn.shape
    out = np.zeros((batch, heads * rot), dtype=np.float32)
    lib().orc_kqv(_p(out), _p(vcache), _p(attn), backlog, heads, rot, batch)
    return out


def attention(kcache, vcache, q, pos, heads, rot):
    """mhsa -> softmax -> kqv, the chain of llava_layer.cpp:59-62"""
    return kqv(vcache, softmax(mhsa(kcache, q, pos, heads, rot), pos, rot), heads, rot)


def num_threads():
    return int(lib().orc_num_threads())


def greedy(logits):
    logits = _f32(logits)
    return int(lib().orc_sample_greedy(_p(logits), logits.shape[0]))


class Model:
    def __init__(self, path):
        self.h = lib().orc_model_open(os.fsencode(path))
        if not self.h:
            raise ValueError(f"oracle cannot parse {path}")
        hp = HParams()
        lib().orc_model_hparams(self.h, C.byref(hp))
        self.hp = {k: getattr(hp, k) for k, _ in HParams._fields_}

    def tensor(self, name):
        ft, off, rows, cols, size = C.c_uint32(), C.c_uint64(), C.c_uint32(), C.c_uint32(), C.c_uint64()
        rc = lib().orc_model_tensor(self.h, name.encode(), C.byref(ft), C.byref(off), C.byref(rows), C.byref(cols),
                                    C.byref(size))
        if rc:
            raise KeyError(name)
        return dict(ftype=ft.value, offset=off.value, rows=rows.value, cols=cols.value, size=size.value)

    def data(self, name):
        t = self.tensor(name)
        addr = lib().orc_model_data(self.h, t["offset"])
        return np.ctypeslib.as_array(C.cast(addr, C.POINTER(C.c_uint8)), shape=(t["size"],)), t

    def forward_f64(self, tokens, kv=None, activation_bits=0):
        """logits of the last of `tokens` in double precision (new cache rows still rounded to fp16): the yardstick for
        tolerances between fp32 implementations.  kv = None: a prompt from position 0; else a list with one (k_rows, v_rows)
        pair of uint16 arrays [pos0][dim] per layer, the cache the tokens continue from."""
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        out = np.empty(self.hp["vocab"], dtype=np.float64)
        pos0, kp, vp_ = 0, None, None
        if kv is not None:
            ks = [np.ascontiguousarray(k, dtype=np.uint16) for k, _ in kv]
            vs = [np.ascontiguousarray(v, dtype=np.uint16) for _, v in kv]
            pos0 = ks[0].shape[0]
            assert len(ks) == self.hp["layers"] and all(a.shape == (pos0, self.hp["dim"]) for a in ks + vs)
            kp = (C.c_void_p * len(ks))(*[a.ctypes.data for a in ks])
            vp_ = (C.c_void_p * len(vs))(*[a.ctypes.data for a in vs])
        lib().orc_forward_f64_activation_bits(activation_bits)   # > 0: GEMM inputs quantised per block to that many bits (experiment)
        rc = lib().orc_forward_f64(self.h, _p(t), t.shape[0], pos0, kp, vp_, _p(out))
        lib().orc_forward_f64_activation_bits(0)
        if rc:
            raise ValueError(f"orc_forward_f64 failed ({rc})")
        return out

    def close(self):
        if self.h:
            lib().orc_model_close(self.h)
            self.h = None


class Session:
    def __init__(self, model, backlog=128):
        self.model = model
        self.backlog = backlog
        self.h = lib().orc_session_new(model.h, backlog)
        if not self.h:
            raise ValueError("oracle session: model lacks tensors or backlog is not a power of two")

    @property
    def pos(self):
        return lib().orc_session_pos(self.h)

    def rewind(self, pos):
        lib().orc_session_rewind(self.h, pos)

    def eval(self, tokens, all_rows=False):
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        V = self.model.hp["vocab"]
        last = np.empty(V, dtype=np.float32)
        every = np.empty((t.shape[0], V), dtype=np.float32) if all_rows else None
        rc = lib().orc_session_eval(self.h, _p(t), t.shape[0], _p(last), _p(every) if all_rows else None)
        if rc:
            raise ValueError(f"orc_session_eval failed ({rc})")
        return every if all_rows else last

    def kv(self, layer, which, n_tokens):
        addr = lib().orc_session_kv(self.h, layer, which)
        D = self.model.hp["dim"]
        full = np.ctypeslib.as_array(C.cast(addr, C.POINTER(C.c_uint16)), shape=(self.backlog, D))
        return full[:n_tokens].copy()

    def kv_load(self, layer, which, rows):
        rows = np.ascontiguousarray(rows, dtype=np.uint16)
        if lib().orc_session_kv_load(self.h, layer, which, _p(rows), rows.shape[0]):
            raise ValueError("orc_session_kv_load refused the arguments")

    def set_pos(self, pos):
        if lib().orc_session_set_pos(self.h, pos):
            raise ValueError("position beyond the backlog")

    def trace(self, layer, which):
        n = C.c_uint32()
        addr = lib().orc_session_trace(self.h, layer, which, C.byref(n))
        return np.ctypeslib.as_array(C.cast(addr, C.POINTER(C.c_float)), shape=(n.value,)).copy()

    def close(self):
        if self.h:
            lib().orc_session_free(self.h)
            self.h = None


# ---- the reference's own parser / tokenizer, when it was built here from /root/reference -------------------
_ref = None


def ref_available():
    return os.path.exists(REF_PATH)


def ref():
    global _ref
    if _ref is None:
        R = C.CDLL(REF_PATH)
        R.ref_ggml_open.argtypes = [C.c_char_p]
        R.ref_ggml_open.restype = C.c_void_p
        R.ref_ggml_close.argtypes = [C.c_void_p]
        R.ref_ggml_close.restype = None
        R.ref_ggml_header.argtypes = [C.c_void_p, C.POINTER(C.c_uint)]
        R.ref_ggml_vocab_size.argtypes = [C.c_void_p]
        R.ref_ggml_vocab_size.restype = C.c_uint
        R.ref_ggml_token.argtypes = [C.c_void_p, C.c_uint, C.c_char_p, C.c_uint, C.POINTER(C.c_float)]
        R.ref_ggml_token.restype = C.c_uint
        R.ref_ggml_tensor.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_uint), C.POINTER(C.c_ulonglong),
                                      C.POINTER(C.c_uint), C.POINTER(C.c_uint), C.POINTER(C.c_ulonglong)]
        R.ref_ggml_tensor.restype = None
        R.ref_ggml_tokenize.argtypes = [C.c_void_p, C.c_char_p, C.c_uint, C.c_int, C.POINTER(C.c_uint), C.c_uint]
        R.ref_ggml_tokenize.restype = C.c_uint
        R.ref_ggml_detokenize.argtypes = [C.c_void_p, C.POINTER(C.c_uint), C.c_uint, C.c_char_p, C.c_uint]
        R.ref_ggml_detokenize.restype = C.c_uint
        _ref = R
    return _ref


class RefGgml:
    """The reference's ggml_file class (ggml_file.h:43-57) on a file."""

    def __init__(self, path):
        self.h = ref().ref_ggml_open(os.fsencode(path))
        if not self.h:
            raise ValueError(path)

    def header(self):
        out = (C.c_uint * 9)()
        n = ref().ref_ggml_header(self.h, out)
        keys = ["file_version", "vocab", "dim", "multiple_of", "heads", "layers", "rot", "ftype", "ff"]
        assert n == 9
        return dict(zip(keys, [int(v) for v in out]))

    def tensor(self, name):
        ft, off, s1, s2, size = C.c_uint(), C.c_ulonglong(), C.c_uint(), C.c_uint(), C.c_ulonglong()
        ref().ref_ggml_tensor(self.h, name.encode(), C.byref(ft), C.byref(off), C.byref(s1), C.byref(s2), C.byref(size))
        return dict(ftype=ft.value, offset=off.value, rows=s1.value, cols=s2.value, size=size.value)

    def vocab(self):
        n = ref().ref_ggml_vocab_size(self.h)
        out = []
        buf = C.create_string_buffer(256)
        for i in range(n):
            score = C.c_float()
            ln = ref().ref_ggml_token(self.h, i, buf, 256, C.byref(score))
            out.append((buf.raw[:ln], score.value))
        return out

    def tokenize(self, text: bytes, bos: bool):
        cap = 4 * len(text) + 8
        out = (C.c_uint * cap)()
        n = ref().ref_ggml_tokenize(self.h, text, len(text), int(bos), out, cap)
        return [int(out[i]) for i in range(n)]

    def detokenize(self, ids):
        arr = (C.c_uint * len(ids))(*ids)
        cap = 64 * len(ids) + 8
        buf = C.create_string_buffer(cap)
        n = ref().ref_ggml_detokenize(self.h, arr, len(ids), buf, cap)
        return buf.raw[:n]

    def close(self):
        if self.h:
            ref().ref_ggml_close(self.h)
            self.h = None
