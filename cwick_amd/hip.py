"""ctypes binding of libcwick_hip.so (include/cwick_hip.h), one Python function
per C entry point with the same name, argument meaning and 1/0 convention.

There is no CPU fallback here: if the library is missing the import of any
function raises, and a call that the library declines raises Declined with the
library's own reason (cwick_hip_last_error) unless the caller asks for the raw
return code.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libcwick_hip.so")

KDIM, VDIM, NBLK, BLOCK, IDIM = 576, 512, 5, 128, 128


class Declined(RuntimeError):
    """The GPU backend returned 0: the engine would run its CPU path."""


_lib = None

_u8p, _u16p, _i32p, _f32p = (C.POINTER(C.c_uint8), C.POINTER(C.c_uint16),
                             C.POINTER(C.c_int32), C.POINTER(C.c_float))
_vp, _i64, _int, _flt = C.c_void_p, C.c_int64, C.c_int, C.c_float

# name -> (restype, argtypes); every symbol include/cwick_hip.h declares
SIGNATURES = {
    "cwick_hip_ready": (_int, []),
    "cwick_hip_force": (_int, [_int]),
    "cwick_hip_shutdown": (None, []),
    "cwick_hip_last_error": (C.c_char_p, []),
    "cwick_hip_device_info": (_int, [C.c_char_p, C.c_size_t]),
    "cwick_hip_kv_create": (_vp, [_i64, _int, _int]),
    "cwick_hip_kv_free": (None, [_vp]),
    "cwick_hip_kv_write": (_int, [_vp, _i64, _i64, _vp, _vp]),
    "cwick_hip_kv_write_f32": (_int, [_vp, _i64, _i64, _vp, _vp]),
    "cwick_hip_kv_read": (_int, [_vp, _i64, _i64, _vp, _vp]),
    "cwick_hip_kv_read_f32": (_int, [_vp, _i64, _i64, _vp, _vp]),
    "cwick_hip_kv_k_dev": (_vp, [_vp]),
    "cwick_hip_kv_v_dev": (_vp, [_vp]),
    "cwick_hip_latent_create": (_vp, [_int, _i64]),
    "cwick_hip_latent_free": (None, [_vp]),
    "cwick_hip_latent_write": (_int, [_vp, _int, _i64, _i64, _vp, _vp]),
    "cwick_hip_latent_write_f32": (_int, [_vp, _int, _i64, _i64, _vp]),
    "cwick_hip_latent_read": (_int, [_vp, _int, _i64, _i64, _vp, _vp]),
    "cwick_hip_latent_rows_dev": (_vp, [_vp, _int]),
    "cwick_hip_latent_scales_dev": (_vp, [_vp, _int]),
    "cwick_hip_ikeys_create": (_vp, [_int, _i64]),
    "cwick_hip_ikeys_free": (None, [_vp]),
    "cwick_hip_ikeys_write": (_int, [_vp, _int, _i64, _i64, _vp, _vp]),
    "cwick_hip_ikeys_write_f32": (_int, [_vp, _int, _i64, _i64, _vp]),
    "cwick_hip_ikeys_read": (_int, [_vp, _int, _i64, _i64, _vp, _vp]),
    "cwick_hip_ikeys_rows_dev": (_vp, [_vp, _int]),
    "cwick_hip_ikeys_scales_dev": (_vp, [_vp, _int]),
    "cwick_hip_gqa_decode": (_int, [_vp, _i64, _vp, _int, _flt, _vp]),
    "cwick_hip_gqa_prefill": (_int, [_vp, _i64, _i64, _vp, _int, _flt, _vp]),
    "cwick_hip_mla_decode": (_int, [_vp, _int, _vp, _i64, _vp, _int, _flt, _vp]),
    "cwick_hip_mla_decode_sink": (_int, [_vp, _int, _vp, _i64, _vp, _int, _flt, _vp, _vp]),
    "cwick_hip_mla_prefill_chunk": (_int, [_vp, _int, _i64, _i64, _vp, _int, _flt, _vp]),
    "cwick_hip_indexer_scores": (_int, [_vp, _int, _i64, _vp, _vp, _int, _vp]),
    "cwick_hip_indexer_scores_mode": (_int, [_vp, _int, _i64, _vp, _vp, _int, _int, _vp]),
    "cwick_hip_indexer_scores_approx": (_int, [_vp, _int, _i64, _vp, _vp, _int, _vp, C.POINTER(_flt)]),
    "cwick_hip_topk": (_int, [_vp, _i64, _i64, _vp, C.POINTER(_i64)]),
    "cwick_hip_dsa_decode": (_int, [_vp, _vp, _int, _int, _int, _i64, _vp, _vp, _int, _i64,
                                    _vp, _int, _flt, _vp, _vp]),
    "cwick_hip_gqa_decode_dev": (_int, [_vp, _vp, _i64, _int, _int, _vp, _int, _flt, _vp, _vp]),
    "cwick_hip_gqa_prefill_dev": (_int, [_vp, _vp, _i64, _i64, _int, _int, _vp, _int, _flt,
                                         _vp, _vp]),
    "cwick_hip_mla_decode_dev": (_int, [_vp, _vp, _i64, _i64, _i64, _int, _vp, _i64, _vp, _int,
                                        _flt, _vp, _vp]),
    "cwick_hip_mla_decode_static_dev": (_int, [_vp, _vp, _i64, _i64, _i64, _int, _vp, _i64, _vp, _int,
                                               _flt, _vp, _vp]),
    "cwick_hip_mla_decode_sink_dev": (_int, [_vp, _vp, _i64, _i64, _i64, _int, _vp, _i64, _vp, _int,
                                             _flt, _vp, _vp, _vp]),
    "cwick_hip_mla_prefill_chunk_dev": (_int, [_vp, _vp, _i64, _i64, _vp, _int, _flt, _vp, _vp]),
    "cwick_hip_indexer_scores_dev": (_int, [_vp, _vp, _i64, _i64, _int, _i64, _vp, _vp, _int,
                                            _vp, _vp]),
    "cwick_hip_indexer_scores_mode_dev": (_int, [_vp, _vp, _i64, _i64, _int, _i64, _vp, _vp, _int,
                                                 _int, _vp, _vp]),
    "cwick_hip_topk_dev": (_int, [_vp, _int, _i64, _i64, _vp, _vp]),
    "cwick_hip_dsa_decode_dev": (_int, [_vp, _vp, _i64, _i64, _vp, _vp, _i64, _i64, _int, _i64,
                                        _vp, _vp, _int, _i64, _vp, _int, _flt, _vp, _vp, _vp,
                                        _vp]),
    "cwick_hip_mla_absorb_dev": (_int, [_vp, _vp, _i64, _int, _int, _int, _int, _int, _int, _int, _vp, _vp]),
    "cwick_hip_mla_expand_dev": (_int, [_vp, _vp, _int, _int, _int, _int, _int, _int, _vp, _vp]),
    "cwick_hip_gqa_prepare_dev": (_int, [_vp, _i64, _vp, _vp, _i64, _i64, _int, _int, _int, _vp, _vp, _flt,
                                         _vp, _vp, _int, _vp, _vp, _vp]),
    "cwick_hip_gqa_decode_sel": (_int, [_vp, _vp, _i64, _vp, _int, _flt, _vp]),
    "cwick_hip_gqa_decode_sel_dev": (_int, [_vp, _vp, _i64, _int, _int, _vp, _i64, _vp, _int, _flt, _vp, _vp]),
    "cwick_hip_ikeys_pool_append_dev": (_int, [_vp, _int, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _flt, _int, _vp, _vp]),
    "cwick_hip_candidate_select_dev": (_int, [_vp, _int, _i64, _int, _i64, _vp, _vp]),
    "cwick_hip_candidate_apply_dev": (_int, [_vp, _vp, _int, _i64, _vp]),
    "cwick_hip_glm_select_dev": (_int, [_vp, _int, _i64, _i64, _int, _i64, _int, _vp, _i64, _vp, _vp]),
    "cwick_hip_mm_select": (_int, [_vp, _i64, _vp, _int, _int, _int, _vp, _vp, _i64, _vp]),
    "cwick_hip_mm_select_dev": (_int, [_vp, _vp, _int, _i64, _int, _int, _int, _int, _vp, _i64, _vp, _vp, _i64, _vp, _vp]),
    "cwick_hip_latent_read_f32": (_int, [_vp, _int, _i64, _i64, _vp]),
    "cwick_hip_ikeys_read_f32": (_int, [_vp, _int, _i64, _i64, _vp]),
    "cwick_hip_reserve_dev": (_int, [_vp, _i64]),
    "cwick_hip_workspace_bytes_dev": (_i64, [_vp]),
    "cwick_hip_stream_release": (_int, [_vp]),
    "cwick_hip_probe_hbm_read": (_int, [C.c_size_t, _int, C.POINTER(C.c_double)]),
    "cwick_hip_probe_mfma": (_int, [_int, _int, C.POINTER(C.c_double)]),
    "cwick_hip_e4m3_table": (_int, [_vp]),
    "cwick_hip_lane_ops": (_int, [_vp, _vp]),
    "cwick_hip_prof_enable": (None, [_int]),
    "cwick_hip_prof_reset": (None, []),
    "cwick_hip_prof_read": (_int, [_int, C.POINTER(C.c_double), C.POINTER(_i64)]),
    "cwick_hip_prof_name": (C.c_char_p, [_int]),
}


def lib():
    """Load libcwick_hip.so.  Raises if it has not been built: nothing in this
    package computes attention any other way."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: build it with `python -m cwick_amd.build` (hipcc, gfx950)"
                % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def last_error():
    return lib().cwick_hip_last_error().decode("utf-8", "replace")


def _check(rc, what):
    if rc != 1:
        raise Declined("%s declined: %s" % (what, last_error()))
    return rc


def ready():
    return lib().cwick_hip_ready() == 1


def force(on):
    return lib().cwick_hip_force(1 if on else 0)


def shutdown():
    lib().cwick_hip_shutdown()


def device_info():
    buf = C.create_string_buffer(256)
    if lib().cwick_hip_device_info(buf, 256) != 1:
        raise Declined("device_info: " + last_error())
    return buf.value.decode()


def _np(a, dtype):
    a = np.ascontiguousarray(a, dtype)
    return a, a.ctypes.data


def _dp(t):
    """Device address of a torch tensor (or a raw integer address / None)."""
    if t is None:
        return None
    if isinstance(t, int):
        return t
    assert t.is_cuda and t.is_contiguous()
    return t.data_ptr()


# ------------------------------------------------------------------ caches
class KVCache:
    """cwick_hip_kv: bf16 K/V rows [capacity][n_kv_heads*head_dim] in HBM."""

    def __init__(self, capacity, n_kv_heads, head_dim):
        self.capacity, self.n_kv_heads, self.head_dim = capacity, n_kv_heads, head_dim
        self.h = lib().cwick_hip_kv_create(capacity, n_kv_heads, head_dim)
        if not self.h:
            raise Declined("kv_create: " + last_error())

    def write(self, pos0, k_rows, v_rows):
        k, kp = _np(k_rows, np.uint16)
        v, vp = _np(v_rows, np.uint16)
        n = k.shape[0]
        _check(lib().cwick_hip_kv_write(self.h, pos0, n, kp, vp), "kv_write")

    def write_f32(self, pos0, k_rows, v_rows):
        k, kp = _np(k_rows, np.float32)
        v, vp = _np(v_rows, np.float32)
        _check(lib().cwick_hip_kv_write_f32(self.h, pos0, k.shape[0], kp, vp), "kv_write_f32")

    def read(self, pos0, n):
        row = self.n_kv_heads * self.head_dim
        k = np.empty((n, row), np.uint16)
        v = np.empty((n, row), np.uint16)
        _check(lib().cwick_hip_kv_read(self.h, pos0, n, k.ctypes.data, v.ctypes.data), "kv_read")
        return k, v

    def read_f32(self, pos0, n):
        row = self.n_kv_heads * self.head_dim
        k = np.empty((n, row), np.float32)
        v = np.empty((n, row), np.float32)
        _check(lib().cwick_hip_kv_read_f32(self.h, pos0, n, k.ctypes.data, v.ctypes.data), "kv_read_f32")
        return k, v

    def k_dev(self):
        return lib().cwick_hip_kv_k_dev(self.h)

    def v_dev(self):
        return lib().cwick_hip_kv_v_dev(self.h)

    def free(self):
        if self.h:
            lib().cwick_hip_kv_free(self.h)
            self.h = None

    __del__ = free


class LatentCache:
    """cwick_hip_latent: FP8 rows [slots][capacity][576] + scales [..][5]."""

    def __init__(self, slots, capacity):
        self.slots, self.capacity = slots, capacity
        self.h = lib().cwick_hip_latent_create(slots, capacity)
        if not self.h:
            raise Declined("latent_create: " + last_error())

    def write(self, slot, pos0, rows, scales):
        r, rp = _np(rows, np.uint8)
        s, sp = _np(scales, np.float32)
        assert r.shape[1] == KDIM and s.shape == (r.shape[0], NBLK)
        _check(lib().cwick_hip_latent_write(self.h, slot, pos0, r.shape[0], rp, sp), "latent_write")

    def write_f32(self, slot, pos0, rows):
        r, rp = _np(rows, np.float32)
        assert r.shape[1] == KDIM
        _check(lib().cwick_hip_latent_write_f32(self.h, slot, pos0, r.shape[0], rp),
               "latent_write_f32")

    def read(self, slot, pos0, n):
        rows = np.empty((n, KDIM), np.uint8)
        scales = np.empty((n, NBLK), np.float32)
        _check(lib().cwick_hip_latent_read(self.h, slot, pos0, n, rows.ctypes.data,
                                           scales.ctypes.data), "latent_read")
        return rows, scales

    def read_f32(self, slot, pos0, n):
        rows = np.empty((n, KDIM), np.float32)
        _check(lib().cwick_hip_latent_read_f32(self.h, slot, pos0, n, rows.ctypes.data), "latent_read_f32")
        return rows

    def rows_dev(self, slot=0):
        return lib().cwick_hip_latent_rows_dev(self.h, slot)

    def scales_dev(self, slot=0):
        return lib().cwick_hip_latent_scales_dev(self.h, slot)

    def free(self):
        if self.h:
            lib().cwick_hip_latent_free(self.h)
            self.h = None

    __del__ = free


class IndexKeys:
    """cwick_hip_ikeys: FP8 indexer keys [slots][capacity][128] + scale per token."""

    def __init__(self, slots, capacity):
        self.slots, self.capacity = slots, capacity
        self.h = lib().cwick_hip_ikeys_create(slots, capacity)
        if not self.h:
            raise Declined("ikeys_create: " + last_error())

    def write(self, slot, pos0, rows, scales):
        r, rp = _np(rows, np.uint8)
        s, sp = _np(scales, np.float32)
        assert r.shape[1] == IDIM and s.size == r.shape[0]
        _check(lib().cwick_hip_ikeys_write(self.h, slot, pos0, r.shape[0], rp, sp), "ikeys_write")

    def write_f32(self, slot, pos0, rows):
        r, rp = _np(rows, np.float32)
        _check(lib().cwick_hip_ikeys_write_f32(self.h, slot, pos0, r.shape[0], rp),
               "ikeys_write_f32")

    def read(self, slot, pos0, n):
        rows = np.empty((n, IDIM), np.uint8)
        scales = np.empty(n, np.float32)
        _check(lib().cwick_hip_ikeys_read(self.h, slot, pos0, n, rows.ctypes.data,
                                          scales.ctypes.data), "ikeys_read")
        return rows, scales

    def read_f32(self, slot, pos0, n):
        rows = np.empty((n, IDIM), np.float32)
        _check(lib().cwick_hip_ikeys_read_f32(self.h, slot, pos0, n, rows.ctypes.data), "ikeys_read_f32")
        return rows

    def pool_append_dev(self, slot, pos0, n, raw_k, raw_gate, ape, k_norm_w, k_norm_b, eps, kpool,
                        rows_f32=None, stream=None, raw=False):
        """Device operands (torch tensors): close n pools and store their keys as rows pos0.."""
        rc = lib().cwick_hip_ikeys_pool_append_dev(self.h, slot, pos0, n, _dp(raw_k), _dp(raw_gate), _dp(ape),
                                                   _dp(k_norm_w), _dp(k_norm_b), eps, kpool, _dp(rows_f32), stream)
        return rc if raw else _check(rc, "ikeys_pool_append_dev")

    def rows_dev(self, slot=0):
        return lib().cwick_hip_ikeys_rows_dev(self.h, slot)

    def scales_dev(self, slot=0):
        return lib().cwick_hip_ikeys_scales_dev(self.h, slot)

    def free(self):
        if self.h:
            lib().cwick_hip_ikeys_free(self.h)
            self.h = None

    __del__ = free


# ------------------------------------------------------------------ host-pointer ops
def gqa_decode(cache, n_keys, q, scale, raw=False):
    q, qp = _np(q, np.uint16)
    nh, hd = q.shape
    out = np.empty((nh, hd), np.float32)
    rc = lib().cwick_hip_gqa_decode(cache.h, n_keys, qp, nh, scale, out.ctypes.data)
    if raw:
        return rc, out
    _check(rc, "gqa_decode")
    return out


def gqa_decode_sel(cache, sel, q, scale, raw=False):
    q, qp = _np(q, np.uint16)
    sel, sp = _np(sel, np.int32)
    nh, hd = q.shape
    out = np.empty((nh, hd), np.float32)
    rc = lib().cwick_hip_gqa_decode_sel(cache.h, sp, sel.size, qp, nh, scale, out.ctypes.data)
    if raw:
        return rc, out
    _check(rc, "gqa_decode_sel")
    return out


def gqa_decode_sel_dev(k, v, n_rows, n_kv_heads, head_dim, sel, n_list, q, n_heads, scale, out, stream=None):
    return _check(lib().cwick_hip_gqa_decode_sel_dev(_dp(k), _dp(v), n_rows, n_kv_heads, head_dim, _dp(sel), n_list,
                                                     _dp(q), n_heads, scale, _dp(out), stream), "gqa_decode_sel_dev")


def gqa_prefill(cache, pos0, q, scale, raw=False):
    q, qp = _np(q, np.uint16)
    n, nh, hd = q.shape
    out = np.empty((n, nh, hd), np.float32)
    rc = lib().cwick_hip_gqa_prefill(cache.h, pos0, n, qp, nh, scale, out.ctypes.data)
    if raw:
        return rc, out
    _check(rc, "gqa_prefill")
    return out


def mla_decode(cache, slot, q, scale, sel=None, n_list=None, raw=False, sink=None):
    q, qp = _np(q, np.uint16)
    nh = q.shape[0]
    assert q.shape[1] == KDIM
    selp = None
    if sel is not None:
        sel, selp = _np(sel, np.int32)
        n_list = sel.size if n_list is None else n_list
    out = np.empty((nh, VDIM), np.float32)
    if sink is not None:
        sink, sinkp = _np(sink, np.float32)
        assert sink.size == nh
        rc = lib().cwick_hip_mla_decode_sink(cache.h, slot, selp, n_list, qp, nh, scale, sinkp,
                                             out.ctypes.data)
    else:
        rc = lib().cwick_hip_mla_decode(cache.h, slot, selp, n_list, qp, nh, scale, out.ctypes.data)
    if raw:
        return rc, out
    _check(rc, "mla_decode")
    return out


def mla_prefill_chunk(cache, slot, pos0, q, scale, raw=False):
    q, qp = _np(q, np.uint16)
    n, nh, kd = q.shape
    assert kd == KDIM
    out = np.empty((n, nh, VDIM), np.float32)
    rc = lib().cwick_hip_mla_prefill_chunk(cache.h, slot, pos0, n, qp, nh, scale, out.ctypes.data)
    if raw:
        return rc, out
    _check(rc, "mla_prefill_chunk")
    return out


INDEXER_GLM, INDEXER_DS = 0, 1


def indexer_scores(ikeys, slot, n_keys, q_idx, w, raw=False, mode=None):
    q, qp = _np(q_idx, np.uint16)
    w, wp = _np(w, np.float32)
    ih = q.shape[0]
    out = np.empty(n_keys, np.float32)
    if mode is None:
        rc = lib().cwick_hip_indexer_scores(ikeys.h, slot, n_keys, qp, wp, ih, out.ctypes.data)
    else:
        rc = lib().cwick_hip_indexer_scores_mode(ikeys.h, slot, n_keys, qp, wp, ih, mode,
                                                 out.ctypes.data)
    if raw:
        return rc, out
    _check(rc, "indexer_scores")
    return out


def indexer_scores_approx(ikeys, slot, n_keys, q_idx, w):
    """(approximate scores, bound): |approximate - exact| <= bound for every key of the row."""
    q, qp = _np(q_idx, np.uint16)
    w, wp = _np(w, np.float32)
    out = np.empty(n_keys, np.float32)
    bound = _flt(0.0)
    _check(lib().cwick_hip_indexer_scores_approx(ikeys.h, slot, n_keys, qp, wp, q.shape[0],
                                                 out.ctypes.data, C.byref(bound)), "indexer_scores_approx")
    return out, float(bound.value)


def topk(scores, k, raw=False):
    s, sp = _np(scores, np.float32)
    out = np.empty(max(k, 1), np.int32)
    got = _i64(0)
    rc = lib().cwick_hip_topk(sp, s.size, k, out.ctypes.data, C.byref(got))
    if raw:
        return rc, out[:got.value]
    _check(rc, "topk")
    return out[:got.value].copy()


def dsa_decode(ikeys, latent, slot0, slot_step, n_keys, q_idx, w, topk_k, q, scale, raw=False):
    qi, qip = _np(q_idx, np.uint16)
    w, wp = _np(w, np.float32)
    q, qp = _np(q, np.uint16)
    batch, ih, _ = qi.shape
    nh = q.shape[1]
    out = np.empty((batch, nh, VDIM), np.float32)
    sel = np.empty((batch, topk_k), np.int32)
    rc = lib().cwick_hip_dsa_decode(ikeys.h, latent.h, slot0, slot_step, batch, n_keys, qip, wp,
                                    ih, topk_k, qp, nh, scale, out.ctypes.data, sel.ctypes.data)
    if raw:
        return rc, out, sel
    _check(rc, "dsa_decode")
    return out, sel


def probe_hbm_read(nbytes=4 << 30, reps=5):
    """Measured read ceiling of the device in GB/s (128-bit grid-stride read)."""
    v = C.c_double(0.0)
    _check(lib().cwick_hip_probe_hbm_read(nbytes, reps, C.byref(v)), "probe_hbm_read")
    return v.value


def probe_mfma(kind=0, reps=3):
    """Measured matrix-core ceiling in TFLOP/s: kind 0 bf16 32x32x16, kind 1 FP8 16x16x128."""
    v = C.c_double(0.0)
    _check(lib().cwick_hip_probe_mfma(kind, reps, C.byref(v)), "probe_mfma")
    return v.value


def lane_ops(words):
    """The wave-level exchange primitives applied to 64 words: [13][64] uint32 (see cwick_hip.h)."""
    w = np.ascontiguousarray(words, dtype=np.uint32)
    assert w.shape == (64,)
    out = np.empty((13, 64), np.uint32)
    _check(lib().cwick_hip_lane_ops(w.ctypes.data, out.ctypes.data), "lane_ops")
    return out


def e4m3_table():
    out = np.empty(256, np.float32)
    _check(lib().cwick_hip_e4m3_table(out.ctypes.data), "e4m3_table")
    return out


# ------------------------------------------------------------------ HBM-resident ops
# Arguments are torch CUDA tensors (or raw device addresses); `stream` is a raw
# hipStream_t address (torch.cuda.current_stream().cuda_stream) or None.
def gqa_decode_dev(k, v, n_keys, n_kv_heads, head_dim, q, n_heads, scale, out, stream=None):
    return _check(lib().cwick_hip_gqa_decode_dev(_dp(k), _dp(v), n_keys, n_kv_heads, head_dim,
                                                 _dp(q), n_heads, scale, _dp(out), stream),
                  "gqa_decode_dev")


def gqa_prefill_dev(k, v, pos0, n, n_kv_heads, head_dim, q, n_heads, scale, out, stream=None):
    return _check(lib().cwick_hip_gqa_prefill_dev(_dp(k), _dp(v), pos0, n, n_kv_heads, head_dim,
                                                  _dp(q), n_heads, scale, _dp(out), stream),
                  "gqa_prefill_dev")


def mla_decode_dev(rows, scales, row_bstride, scale_bstride, n_rows, batch, sel, n_list, q,
                   n_heads, scale, out, stream=None, raw=False):
    rc = lib().cwick_hip_mla_decode_dev(_dp(rows), _dp(scales), row_bstride, scale_bstride, n_rows, batch,
                                        _dp(sel), n_list, _dp(q), n_heads, scale, _dp(out), stream)
    return rc if raw else _check(rc, "mla_decode_dev")


def mla_decode_static_dev(rows, scales, row_bstride, scale_bstride, n_rows, batch, sel, n_list, q,
                          n_heads, scale, out, stream=None, raw=False):
    """cwick_hip_mla_decode_dev that allocates nothing (fixed scratch inside the library)."""
    rc = lib().cwick_hip_mla_decode_static_dev(_dp(rows), _dp(scales), row_bstride, scale_bstride,
                                               n_rows, batch, _dp(sel), n_list, _dp(q), n_heads,
                                               scale, _dp(out), stream)
    return rc if raw else _check(rc, "mla_decode_static_dev")


def mla_prefill_chunk_dev(rows, scales, pos0, n, q, n_heads, scale, out, stream=None):
    return _check(lib().cwick_hip_mla_prefill_chunk_dev(_dp(rows), _dp(scales), pos0, n, _dp(q),
                                                        n_heads, scale, _dp(out), stream),
                  "mla_prefill_chunk_dev")


def indexer_scores_dev(keys, kscale, key_bstride, kscale_bstride, batch, n_keys, q_idx, w,
                       n_idx_heads, scores, stream=None):
    return _check(lib().cwick_hip_indexer_scores_dev(_dp(keys), _dp(kscale), key_bstride,
                                                     kscale_bstride, batch, n_keys, _dp(q_idx),
                                                     _dp(w), n_idx_heads, _dp(scores), stream),
                  "indexer_scores_dev")


def topk_dev(scores, batch, n, k, out_idx, stream=None):
    return _check(lib().cwick_hip_topk_dev(_dp(scores), batch, n, k, _dp(out_idx), stream),
                  "topk_dev")


def dsa_decode_dev(ikeys, ikscale, key_bstride, kscale_bstride, rows, scales, row_bstride,
                   scale_bstride, batch, n_keys, q_idx, w, n_idx_heads, topk_k, q, n_heads, scale,
                   scores_tmp, sel_out, out, stream=None):
    return _check(lib().cwick_hip_dsa_decode_dev(
        _dp(ikeys), _dp(ikscale), key_bstride, kscale_bstride, _dp(rows), _dp(scales),
        row_bstride, scale_bstride, batch, n_keys, _dp(q_idx), _dp(w), n_idx_heads, topk_k,
        _dp(q), n_heads, scale, _dp(scores_tmp), _dp(sel_out), _dp(out), stream),
        "dsa_decode_dev")


def mla_absorb_dev(kv_b_proj, q, q_bstride, batch, n_heads, q_dim, nope, rope, kv_dim, kv_lora, q_abs,
                   stream=None):
    return _check(lib().cwick_hip_mla_absorb_dev(_dp(kv_b_proj), _dp(q), q_bstride, batch, n_heads, q_dim,
                                                 nope, rope, kv_dim, kv_lora, _dp(q_abs), stream),
                  "mla_absorb_dev")


def mla_expand_dev(kv_b_proj, c_acc, batch, n_heads, nope, vdim, kv_dim, kv_lora, out, stream=None):
    return _check(lib().cwick_hip_mla_expand_dev(_dp(kv_b_proj), _dp(c_acc), batch, n_heads, nope, vdim,
                                                 kv_dim, kv_lora, _dp(out), stream), "mla_expand_dev")


def gqa_prepare_dev(q_proj, q_head_stride, k_proj, v_proj, n, pos0, n_heads, n_kv_heads, head_dim,
                    q_norm, k_norm, eps, rope_cos, rope_sin, rotary_dim, q_out, cache, stream=None, raw=False):
    rc = lib().cwick_hip_gqa_prepare_dev(_dp(q_proj), q_head_stride, _dp(k_proj), _dp(v_proj), n, pos0,
                                         n_heads, n_kv_heads, head_dim, _dp(q_norm), _dp(k_norm), eps,
                                         _dp(rope_cos), _dp(rope_sin), rotary_dim, _dp(q_out), cache.h, stream)
    return rc if raw else _check(rc, "gqa_prepare_dev")


def candidate_select_dev(scores, batch, n, block, keep_blocks, cand, stream=None, raw=False):
    rc = lib().cwick_hip_candidate_select_dev(_dp(scores), batch, n, block, keep_blocks, _dp(cand), stream)
    return rc if raw else _check(rc, "candidate_select_dev")


def mm_select(idx_cache, limit, iq, block, keep_blocks, max_sel):
    """One query, host operands: -> (blocks, positions) as the reference leaves them."""
    iq, iqp = _np(iq, np.float32)
    blk = np.empty(keep_blocks + 1, np.int32)
    sel = np.empty(max_sel, np.int32)
    ns = _i64(0)
    _check(lib().cwick_hip_mm_select(idx_cache.h, limit, iqp, iq.shape[0], block, keep_blocks, blk.ctypes.data,
                                     sel.ctypes.data, max_sel, C.byref(ns)), "mm_select")
    return blk[blk >= 0], sel[:ns.value]


def mm_select_dev(idx_keys, iq, batch, limit0, index_heads, index_dim, block, keep_blocks, scores, score_stride,
                  blk_out, sel, max_sel, n_sel, stream=None, raw=False):
    rc = lib().cwick_hip_mm_select_dev(_dp(idx_keys), _dp(iq), batch, limit0, index_heads, index_dim, block,
                                       keep_blocks, _dp(scores), score_stride, _dp(blk_out), _dp(sel), max_sel,
                                       _dp(n_sel), stream)
    return rc if raw else _check(rc, "mm_select_dev")


def reserve_dev(stream, nbytes, raw=False):
    rc = lib().cwick_hip_reserve_dev(stream, nbytes)
    return rc if raw else _check(rc, "reserve_dev")


def workspace_bytes_dev(stream):
    return int(lib().cwick_hip_workspace_bytes_dev(stream))


def stream_release(stream, raw=False):
    rc = lib().cwick_hip_stream_release(stream)
    return rc if raw else _check(rc, "stream_release")


def glm_select_dev(scores, batch, n_comp, npos, kpool, topk, strict, sel, max_sel, n_sel, stream=None, raw=False):
    rc = lib().cwick_hip_glm_select_dev(_dp(scores), batch, n_comp, npos, kpool, topk, 1 if strict else 0, _dp(sel),
                                        max_sel, _dp(n_sel), stream)
    return rc if raw else _check(rc, "glm_select_dev")


def candidate_apply_dev(scores, cand, batch, n, stream=None):
    return _check(lib().cwick_hip_candidate_apply_dev(_dp(scores), _dp(cand), batch, n, stream),
                  "candidate_apply_dev")


# ------------------------------------------------------------------ phase timers
PROF_NAMES = ["gqa_decode_split_kernel", "splitk_merge_wide_kernel<gqa>", "gqa_prefill_kernel",
              "mla_roles_kernel", "mla_merge_frag16_kernel", "indexer kernels", "topk kernels", "mla_prefill64_kernel",
              "mm select kernels", "indexer_approx_kernel"]


def prof_enable(on=True):
    lib().cwick_hip_prof_enable(1 if on else 0)


def prof_reset():
    lib().cwick_hip_prof_reset()


def prof_read():
    """{kernel name: (total_ms, launches)} since the last reset (waits for the GPU)."""
    out = {}
    for i, name in enumerate(PROF_NAMES):
        ms, n = C.c_double(0.0), _i64(0)
        _check(lib().cwick_hip_prof_read(i, C.byref(ms), C.byref(n)), "prof_read")
        assert lib().cwick_hip_prof_name(i).decode() == name
        out[name] = (ms.value, n.value)
    return out
