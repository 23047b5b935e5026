"""ctypes front end of the CPU oracle (oracle/cwick_oracle.c) and of oracle/_ref.

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg as the checker / reported CPU baseline.  The shipped
package (cwick_amd) never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libcwick_oracle.so")
_REF = os.path.join(_HERE, "_ref", "libcwick_ref.so")

KDIM, VDIM, BLOCK = 576, 512, 128


def build(force=False):
    """Compile the restatement (and _ref when the reference tree is present)."""
    if force or not os.path.exists(_LIB):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []))
    return _LIB


_lib = None
_ref = None


def _p(a, ct):
    return a.ctypes.data_as(C.POINTER(ct))


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            build()
        L = C.CDLL(_LIB)
        L.orc_bf16_to_f32.restype = C.c_float
        L.orc_bf16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_bf16_rne.restype = C.c_uint16
        L.orc_f32_to_bf16_rne.argtypes = [C.c_float]
        L.orc_f32_to_bf16_cwick.restype = C.c_uint16
        L.orc_f32_to_bf16_cwick.argtypes = [C.c_float]
        L.orc_bf16_round.restype = C.c_float
        L.orc_bf16_round.argtypes = [C.c_float]
        L.orc_e4m3_to_f32.restype = C.c_float
        L.orc_e4m3_to_f32.argtypes = [C.c_uint8]
        L.orc_f32_to_e4m3.restype = C.c_uint8
        L.orc_f32_to_e4m3.argtypes = [C.c_float]
        L.orc_f32_to_e4m3_rne.restype = C.c_uint8
        L.orc_f32_to_e4m3_rne.argtypes = [C.c_float]
        L.orc_dot_f32.restype = C.c_float
        L.orc_topk_contract.restype = C.c_int64
        L.orc_topk_quickselect.restype = C.c_int64
        L.orc_topk_heap.restype = C.c_int
        L.orc_topk_order_key.restype = C.c_uint32
        L.orc_topk_order_key.argtypes = [C.c_float]
        L.orc_now_ns.restype = C.c_int64
        L.orc_max_threads.restype = C.c_int
        _lib = L
    return _lib


def ref():
    """The reference's own object code (oracle/_ref), or None if it was not built."""
    global _ref
    if _ref is None and os.path.exists(_REF):
        R = C.CDLL(_REF)
        R.cwick_fp8_e4m3_to_f32.restype = C.c_float
        R.cwick_fp8_e4m3_to_f32.argtypes = [C.c_uint8]
        R.cwick_bf16_to_f32.restype = C.c_float
        R.cwick_bf16_to_f32.argtypes = [C.c_uint16]
        R.cwick_f32_to_bf16.restype = C.c_uint16
        R.cwick_f32_to_bf16.argtypes = [C.c_float]
        R.ds_bf16_round.restype = C.c_float
        R.ds_bf16_round.argtypes = [C.c_float]
        R.ds_topk_scores.restype = C.c_int
        _ref = R
    return _ref


def max_threads():
    return int(lib().orc_max_threads())


# ---------------------------------------------------------------- codecs
def e4m3_lut():
    out = np.empty(256, np.float32)
    lib().orc_e4m3_lut(_p(out, C.c_float))
    return out


def quantize_rows_e4m3(x, block):
    x = np.ascontiguousarray(x, np.float32)
    rows, cols = x.shape
    nb = (cols + block - 1) // block
    q = np.empty((rows, cols), np.uint8)
    s = np.empty((rows, nb), np.float32)
    lib().orc_quantize_rows_e4m3(_p(x, C.c_float), C.c_int64(rows), C.c_int64(cols),
                                 C.c_int64(block), _p(q, C.c_uint8), _p(s, C.c_float))
    return q, s


def softmax(x):
    x = np.array(x, np.float32, copy=True)
    lib().orc_softmax(_p(x, C.c_float), C.c_int64(x.size))
    return x


def dot_f32(a, b):
    a = np.ascontiguousarray(a, np.float32)
    b = np.ascontiguousarray(b, np.float32)
    return float(lib().orc_dot_f32(_p(a, C.c_float), _p(b, C.c_float), C.c_int64(a.size)))


# ---------------------------------------------------------------- attention
def gqa_decode(q, k, v, scale, nslice=16, nthreads=1):
    """q [nh,hd] u16, k/v [keys,nkv,hd] u16 -> [nh,hd] f32."""
    q = np.ascontiguousarray(q, np.uint16)
    k = np.ascontiguousarray(k, np.uint16)
    v = np.ascontiguousarray(v, np.uint16)
    nh, hd = q.shape
    keys, nkv, _ = k.shape
    out = np.empty((nh, hd), np.float32)
    lib().orc_gqa_decode(_p(q, C.c_uint16), _p(k, C.c_uint16), _p(v, C.c_uint16),
                         C.c_int64(keys), nh, nkv, hd, C.c_float(scale), nslice, nthreads,
                         _p(out, C.c_float))
    return out


def gqa_prefill(q, k, v, pos0, scale, tile_q=128, tiles=(0, 0, 1), nthreads=1, out=None):
    """q [n,nh,hd] u16, k/v [pos0+n,nkv,hd] u16 -> [n,nh,hd] f32 (causal)."""
    q = np.ascontiguousarray(q, np.uint16)
    k = np.ascontiguousarray(k, np.uint16)
    v = np.ascontiguousarray(v, np.uint16)
    n, nh, hd = q.shape
    nkv = k.shape[1]
    assert k.shape[0] >= pos0 + n
    if out is None:
        out = np.zeros((n, nh, hd), np.float32)
    lib().orc_gqa_prefill(_p(q, C.c_uint16), _p(k, C.c_uint16), _p(v, C.c_uint16),
                          C.c_int64(pos0), C.c_int64(n), nh, nkv, hd, C.c_float(scale),
                          tile_q, C.c_int64(tiles[0]), C.c_int64(tiles[1]), C.c_int64(tiles[2]),
                          nthreads, _p(out, C.c_float))
    return out


def mla_decode(q, lat, scales, scale, sel=None, nlist=None, nthreads=1,
               kdim=KDIM, vdim=VDIM, block=BLOCK):
    """q [nh,kdim] u16, lat [cap,kdim] u8, scales [cap,nblk] f32 -> [nh,vdim] f32."""
    q = np.ascontiguousarray(q, np.uint16)
    lat = np.ascontiguousarray(lat, np.uint8)
    scales = np.ascontiguousarray(scales, np.float32)
    nh = q.shape[0]
    if sel is not None:
        sel = np.ascontiguousarray(sel, np.int32)
        nlist = sel.size if nlist is None else nlist
        selp = _p(sel, C.c_int32)
    else:
        nlist = lat.shape[0] if nlist is None else nlist
        selp = None
    out = np.empty((nh, vdim), np.float32)
    lib().orc_mla_decode(_p(q, C.c_uint16), _p(lat, C.c_uint8), _p(scales, C.c_float),
                         C.c_int64(kdim), C.c_int64(vdim), C.c_int64(block), selp,
                         C.c_int64(nlist), nh, C.c_float(scale), nthreads, _p(out, C.c_float))
    return out


def mla_decode_f32(q_abs, lat, scale, sel=None, nlist=None):
    q_abs = np.ascontiguousarray(q_abs, np.float32)
    lat = np.ascontiguousarray(lat, np.float32)
    nh, dim = q_abs.shape
    if sel is not None:
        sel = np.ascontiguousarray(sel, np.int64)
        nlist = sel.size
        selp = _p(sel, C.c_int64)
    else:
        nlist = lat.shape[0] if nlist is None else nlist
        selp = None
    out = np.empty((nh, dim), np.float32)
    lib().orc_mla_decode_f32(_p(q_abs, C.c_float), _p(lat, C.c_float), C.c_int64(dim), selp,
                             C.c_int64(nlist), nh, C.c_float(scale), _p(out, C.c_float))
    return out


def mla_prefill_chunk(q, lat, scales, pos0, scale, queries=(0, 0, 1), nthreads=1, out=None,
                      kdim=KDIM, vdim=VDIM, block=BLOCK):
    """q [n,nh,kdim] u16 -> [n,nh,vdim] f32; causal over positions 0..pos0+t."""
    q = np.ascontiguousarray(q, np.uint16)
    lat = np.ascontiguousarray(lat, np.uint8)
    scales = np.ascontiguousarray(scales, np.float32)
    n, nh, _ = q.shape
    assert lat.shape[0] >= pos0 + n
    if out is None:
        out = np.zeros((n, nh, vdim), np.float32)
    lib().orc_mla_prefill_chunk(_p(q, C.c_uint16), _p(lat, C.c_uint8), _p(scales, C.c_float),
                                C.c_int64(kdim), C.c_int64(vdim), C.c_int64(block),
                                C.c_int64(pos0), C.c_int64(n), nh, C.c_float(scale),
                                C.c_int64(queries[0]), C.c_int64(queries[1]),
                                C.c_int64(queries[2]), nthreads, _p(out, C.c_float))
    return out


def indexer_scores(q, w, keys, kscale, n=None, nthreads=1):
    """q [ih,hd] u16, w [ih] f32, keys [n,hd] u8, kscale [n] f32 -> [n] f32."""
    q = np.ascontiguousarray(q, np.uint16)
    w = np.ascontiguousarray(w, np.float32)
    keys = np.ascontiguousarray(keys, np.uint8)
    kscale = np.ascontiguousarray(kscale, np.float32)
    ih, hd = q.shape
    n = keys.shape[0] if n is None else n
    sc = np.empty(n, np.float32)
    lib().orc_indexer_scores(_p(q, C.c_uint16), _p(w, C.c_float), _p(keys, C.c_uint8),
                             _p(kscale, C.c_float), C.c_int64(n), ih, hd, nthreads,
                             _p(sc, C.c_float))
    return sc


def indexer_scores_ds(q, w, keys, kscale, n=None, nthreads=1):
    """ds_indexer's score loop (src/ds_model.c:1099-1121): serial dot, bf16-rounded dot and weight."""
    q = np.ascontiguousarray(q, np.uint16)
    w = np.ascontiguousarray(w, np.float32)
    keys = np.ascontiguousarray(keys, np.uint8)
    kscale = np.ascontiguousarray(kscale, np.float32)
    ih, hd = q.shape
    n = keys.shape[0] if n is None else n
    sc = np.empty(n, np.float32)
    lib().orc_indexer_scores_ds(_p(q, C.c_uint16), _p(w, C.c_float), _p(keys, C.c_uint8),
                                _p(kscale, C.c_float), C.c_int64(n), ih, hd, nthreads,
                                _p(sc, C.c_float))
    return sc


def sparse_attn_sink(q, lat, scales, scale, sink=None, sel=None, nlist=None, nthreads=1,
                     kdim=KDIM, vdim=VDIM, block=BLOCK):
    """ds_sparse_attn_heads (src/ds_model.c:917-966) over the FP8 latent: sink term in the denominator."""
    q = np.ascontiguousarray(q, np.uint16)
    lat = np.ascontiguousarray(lat, np.uint8)
    scales = np.ascontiguousarray(scales, np.float32)
    nh = q.shape[0]
    if sel is not None:
        sel = np.ascontiguousarray(sel, np.int32)
        nlist = sel.size if nlist is None else nlist
        selp = _p(sel, C.c_int32)
    else:
        nlist = lat.shape[0] if nlist is None else nlist
        selp = None
    sinkp = None
    if sink is not None:
        sink = np.ascontiguousarray(sink, np.float32)
        sinkp = _p(sink, C.c_float)
    out = np.empty((nh, vdim), np.float32)
    lib().orc_sparse_attn_sink(_p(q, C.c_uint16), _p(lat, C.c_uint8), _p(scales, C.c_float),
                               C.c_int64(kdim), C.c_int64(vdim), C.c_int64(block), selp,
                               C.c_int64(nlist), nh, C.c_float(scale), sinkp, nthreads,
                               _p(out, C.c_float))
    return out


def mla_absorb(kvb_w, q, nope, rope, kv_dim, kv_lora=512, out_dim=KDIM):
    """q [nh, q_dim] f32, kvb_w [nh*kv_dim, kv_lora] u16 -> q_abs [nh, out_dim] f32."""
    kvb_w = np.ascontiguousarray(kvb_w, np.uint16)
    q = np.ascontiguousarray(q, np.float32)
    nh, q_dim = q.shape
    out = np.empty((nh, out_dim), np.float32)
    lib().orc_mla_absorb(_p(kvb_w, C.c_uint16), _p(q, C.c_float), nh, q_dim, nope, rope, kv_dim, kv_lora,
                         out_dim, _p(out, C.c_float))
    return out


def mla_expand(kvb_w, c_acc, nope, vdim, kv_dim, kv_lora=512):
    kvb_w = np.ascontiguousarray(kvb_w, np.uint16)
    c_acc = np.ascontiguousarray(c_acc, np.float32)
    nh = c_acc.shape[0]
    out = np.empty((nh, vdim), np.float32)
    lib().orc_mla_expand(_p(kvb_w, C.c_uint16), _p(c_acc, C.c_float), nh, nope, vdim, kv_dim, kv_lora,
                         _p(out, C.c_float))
    return out


def build_rope(max_pos, rotary, theta):
    cos_t = np.empty((max_pos, rotary // 2), np.float32)
    sin_t = np.empty((max_pos, rotary // 2), np.float32)
    lib().orc_build_rope(max_pos, rotary, C.c_double(theta), _p(cos_t, C.c_float), _p(sin_t, C.c_float))
    return cos_t, sin_t


def gqa_prepare(q_proj, q_head_stride, k_proj, v_proj, pos0, H, KV, HD, q_norm, k_norm, eps, cos_t, sin_t, rotary):
    q_proj = np.ascontiguousarray(q_proj, np.float32)
    k_proj = np.ascontiguousarray(k_proj, np.float32)
    v_proj = np.ascontiguousarray(v_proj, np.float32)
    n = k_proj.shape[0]
    qo = np.empty((n, H, HD), np.uint16)
    ko = np.empty((n, KV * HD), np.uint16)
    vo = np.empty((n, KV * HD), np.uint16)
    qn = None if q_norm is None else _p(np.ascontiguousarray(q_norm, np.float32), C.c_float)
    kn = None if k_norm is None else _p(np.ascontiguousarray(k_norm, np.float32), C.c_float)
    lib().orc_gqa_prepare(_p(q_proj, C.c_float), C.c_int64(q_head_stride), _p(k_proj, C.c_float),
                          _p(v_proj, C.c_float), C.c_int64(n), C.c_int64(pos0), H, KV, HD, qn, kn,
                          C.c_float(eps), _p(np.ascontiguousarray(cos_t, np.float32), C.c_float),
                          _p(np.ascontiguousarray(sin_t, np.float32), C.c_float), rotary,
                          _p(qo, C.c_uint16), _p(ko, C.c_uint16), _p(vo, C.c_uint16))
    return qo, ko, vo


def indexer_pool_row(tail_k, tail_g, ape_bf16, knw, knb, eps):
    """One compressed indexer key from a closed pool: tail_k, tail_g fp32 [kp][hd], ape bf16 bits."""
    tail_k = np.ascontiguousarray(tail_k, np.float32)
    tail_g = np.ascontiguousarray(tail_g, np.float32)
    ape = np.ascontiguousarray(ape_bf16, np.uint16)
    kp, hd = tail_k.shape
    out = np.empty(hd, np.float32)
    lib().orc_indexer_pool_row(_p(tail_k, C.c_float), _p(tail_g, C.c_float), _p(ape, C.c_uint16),
                               _p(np.ascontiguousarray(knw, np.float32), C.c_float),
                               _p(np.ascontiguousarray(knb, np.float32), C.c_float), C.c_float(eps), kp, hd,
                               _p(out, C.c_float))
    return out


def candidate_mask(scores, block, keep):
    sc = np.ascontiguousarray(scores, np.float32)
    cand = np.empty(sc.size, np.uint8)
    k = lib().orc_candidate_mask(_p(sc, C.c_float), int(sc.size), int(block), int(keep), _p(cand, C.c_uint8))
    return cand, int(k)


def candidate_apply(scores, cand):
    sc = np.array(scores, np.float32, copy=True)
    cd = np.ascontiguousarray(cand, np.uint8)
    lib().orc_candidate_apply(_p(sc, C.c_float), _p(cd, C.c_uint8), int(sc.size))
    return sc


def mm_index_scores(iq, keys, limit=None):
    """iq [ih,id] f32, keys [n,id] bf16 bits -> [limit] f32 (src/mm_model.c:1764-1780)."""
    iq = np.ascontiguousarray(iq, np.float32)
    keys = np.ascontiguousarray(keys, np.uint16)
    ih, idim = iq.shape
    limit = keys.shape[0] if limit is None else int(limit)
    out = np.empty(limit, np.float32)
    lib().orc_mm_index_scores(_p(iq, C.c_float), _p(keys, C.c_uint16), C.c_int64(limit), int(ih), int(idim),
                              _p(out, C.c_float))
    return out


def mm_select_blocks(scores, limit, block, keep, max_sel=4096):
    """-> (blocks, positions) as src/mm_model.c:1733-1761 and :1969-1976 leave them."""
    sc = np.ascontiguousarray(scores, np.float32)
    assert sc.size >= limit
    blk = np.empty(keep + 1, np.int32)
    sel = np.empty(max(max_sel, 1), np.int64)
    ns = C.c_int64(0)
    nb = lib().orc_mm_select_blocks(_p(sc, C.c_float), C.c_int64(limit), int(block), int(keep), _p(blk, C.c_int32),
                                    _p(sel, C.c_int64), C.c_int64(max_sel), C.byref(ns))
    return blk[:nb].copy(), sel[:ns.value].copy()


def topk_contract(sc, k):
    sc = np.ascontiguousarray(sc, np.float32)
    out = np.empty(max(min(k, sc.size), 1), np.int32)
    got = lib().orc_topk_contract(_p(sc, C.c_float), C.c_int64(sc.size), C.c_int64(k),
                                  _p(out, C.c_int32))
    return out[:got].copy()


def topk_heap(sc, k):
    sc = np.ascontiguousarray(sc, np.float32)
    out = np.empty(max(k, 1), np.int32)
    got = lib().orc_topk_heap(_p(sc, C.c_float), int(sc.size), int(k), _p(out, C.c_int32))
    return out[:got].copy()


def topk_quickselect(sc, want):
    sc = np.ascontiguousarray(sc, np.float32)
    out = np.empty(sc.size, np.int32)
    got = lib().orc_topk_quickselect(_p(sc, C.c_float), C.c_int64(sc.size), C.c_int64(want),
                                     _p(out, C.c_int32))
    return out[:got].copy()


def glm_select(sc, npos, kpool, topk, strict=False, faithful=False):
    """indexer_select after the scores (src/attention.c:585-620): the positions kept, or None for
    "the whole prefix".  faithful: the pool choice exactly as the reference makes it; otherwise by
    the contract (the device path)."""
    sc = np.ascontiguousarray(sc, np.float32)
    kp = max(int(kpool), 1)
    want = (topk + kp - 1) // kp
    sel = np.empty((want + 1) * kp + 1, np.int32)
    lib().orc_glm_select.restype = C.c_int64
    got = lib().orc_glm_select(_p(sc, C.c_float), C.c_int64(sc.size), C.c_int64(npos), C.c_int64(kp),
                               C.c_int64(topk), int(bool(strict)), int(bool(faithful)), _p(sel, C.c_int32))
    return None if got < 0 else sel[:got].copy()


def ref_topk_scores(sc, k):
    """ds_topk_scores as compiled from the reference (src/ds_ops.c:310-338)."""
    R = ref()
    sc = np.ascontiguousarray(sc, np.float32)
    out = np.empty(max(k, 1), np.int32)
    heap = np.empty(max(k, 1), np.float32)
    hidx = np.empty(max(k, 1), np.int32)
    got = R.ds_topk_scores(_p(sc, C.c_float), int(sc.size), int(k), _p(out, C.c_int32),
                           _p(heap, C.c_float), _p(hidx, C.c_int32))
    return out[:got].copy()


def now_ns():
    return int(lib().orc_now_ns())
