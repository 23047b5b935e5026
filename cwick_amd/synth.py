"""Seeded synthetic inputs for the five benchmark configurations.

Everything is generated once on the host with numpy's counter-based Philox
generator (seed = 0xC71C + config index unless given), rounded to bf16 with
round-to-nearest-even or quantised to FP8-E4M3 with a per-block fp32 scale
(amax / 448), and the SAME bits are handed to the GPU library and to whatever
checks it.  The codecs here are plain numpy so that input generation does not
depend on the code under test.
"""
import numpy as np

KDIM, VDIM, NBLK, BLOCK, IDIM = 576, 512, 5, 128, 128
SEED0 = 0xC71C


def rng(seed):
    return np.random.Generator(np.random.Philox(seed))


def f32_to_bf16(x):
    """fp32 -> bf16 bits, round to nearest even (the recipe of src/ds_ops.c:89-96)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    u = u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))
    return (u >> np.uint32(16)).astype(np.uint16)


def bf16_to_f32(b):
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def e4m3_table():
    """All 256 E4M3fn values (bias 7, subnormal step 2^-9, 0x7F/0xFF NaN)."""
    b = np.arange(256, dtype=np.uint32)
    e = (b >> 3) & 0xF
    m = (b & 7).astype(np.float32)
    v = np.where(e == 0, m * np.float32(2.0 ** -9),
                 (np.float32(1.0) + m / np.float32(8.0)) *
                 np.exp2(e.astype(np.float32) - np.float32(7.0))).astype(np.float32)
    v = np.where((e == 15) & ((b & 7) == 7), np.float32(np.nan), v)
    return np.where(b >> 7 == 1, -v, v).astype(np.float32)


def f32_to_e4m3(x):
    """fp32 (|x| <= 448) -> E4M3fn byte, round to nearest even."""
    x = np.ascontiguousarray(x, np.float32)
    a = np.abs(x)
    sign = (x.view(np.uint32) >> np.uint32(31)).astype(np.uint8) << np.uint8(7)
    # normal range: round the fp32 mantissa to 3 bits (carry may bump the exponent)
    u = a.view(np.uint32)
    r = u + (np.uint32(0x7FFFF) + ((u >> np.uint32(20)) & np.uint32(1)))
    e = (r >> np.uint32(23)).astype(np.int32) - 127
    m = ((r >> np.uint32(20)) & np.uint32(7)).astype(np.int32)
    normal = ((e + 7) << 3) | m
    normal = np.minimum(normal, 0x7E)                      # saturate at 448
    # subnormal range (below 2^-6): multiples of 2^-9, rint is ties-to-even
    sub = np.rint(a * np.float32(512.0)).astype(np.int32)  # 0..8 (8 == 2^-6 == byte 0x08)
    byte = np.where(a < np.float32(2.0 ** -6), sub, normal).astype(np.uint8)
    return (byte | sign).astype(np.uint8) * (a != 0)


def quantize_rows(x, block):
    """[rows, cols] fp32 -> (bytes [rows, cols], scales [rows, ceil(cols/block)])."""
    x = np.ascontiguousarray(x, np.float32)
    rows, cols = x.shape
    nb = (cols + block - 1) // block
    q = np.empty((rows, cols), np.uint8)
    s = np.empty((rows, nb), np.float32)
    for b in range(nb):
        seg = x[:, b * block:(b + 1) * block]
        amax = np.abs(seg).max(axis=1)
        sc = np.where(amax > 0, amax / np.float32(448.0), np.float32(1.0)).astype(np.float32)
        v = np.clip(seg / sc[:, None], np.float32(-448.0), np.float32(448.0)).astype(np.float32)
        q[:, b * block:(b + 1) * block] = f32_to_e4m3(v)
        s[:, b] = sc
    return q, s


def normal_bf16(g, shape):
    return f32_to_bf16(g.standard_normal(shape, dtype=np.float32))


def latent_cache(g, n_rows, chunk=8192):
    """N(0,1) latent rows quantised to E4M3 with 5 block scales per row."""
    rows = np.empty((n_rows, KDIM), np.uint8)
    scales = np.empty((n_rows, NBLK), np.float32)
    for r0 in range(0, n_rows, chunk):
        r1 = min(n_rows, r0 + chunk)
        x = g.standard_normal((r1 - r0, KDIM), dtype=np.float32)
        rows[r0:r1], scales[r0:r1] = quantize_rows(x, BLOCK)
    return rows, scales


def index_keys(g, n_rows, chunk=16384):
    rows = np.empty((n_rows, IDIM), np.uint8)
    scales = np.empty(n_rows, np.float32)
    for r0 in range(0, n_rows, chunk):
        r1 = min(n_rows, r0 + chunk)
        x = g.standard_normal((r1 - r0, IDIM), dtype=np.float32)
        q, s = quantize_rows(x, IDIM)
        rows[r0:r1], scales[r0:r1] = q, s[:, 0]
    return rows, scales


# ---------------------------------------------------------------- the five configs
def cfg1_gqa_decode(n_keys=4096, nh=16, nkv=4, hd=256, seed=SEED0 + 1):
    g = rng(seed)
    return dict(q=normal_bf16(g, (nh, hd)), k=normal_bf16(g, (n_keys, nkv, hd)),
                v=normal_bf16(g, (n_keys, nkv, hd)), scale=float(1.0 / np.sqrt(hd)),
                n_keys=n_keys, nh=nh, nkv=nkv, hd=hd)


def cfg2_gqa_prefill(n=8192, nh=16, nkv=4, hd=256, pos0=0, seed=SEED0 + 2):
    g = rng(seed)
    return dict(q=normal_bf16(g, (n, nh, hd)), k=normal_bf16(g, (pos0 + n, nkv, hd)),
                v=normal_bf16(g, (pos0 + n, nkv, hd)), scale=float(1.0 / np.sqrt(hd)),
                n=n, pos0=pos0, nh=nh, nkv=nkv, hd=hd)


def cfg3_mla_decode(n_keys=32768, nh=128, seed=SEED0 + 3):
    g = rng(seed)
    rows, scales = latent_cache(g, n_keys)
    return dict(q=normal_bf16(g, (nh, KDIM)), rows=rows, scales=scales,
                scale=float(1.0 / np.sqrt(192.0)), n_keys=n_keys, nh=nh)


def cfg4_mla_prefill(n=4096, pos0=28672, nh=128, seed=SEED0 + 4):
    g = rng(seed)
    rows, scales = latent_cache(g, pos0 + n)
    return dict(q=normal_bf16(g, (n, nh, KDIM)), rows=rows, scales=scales,
                scale=float(1.0 / np.sqrt(192.0)), n=n, pos0=pos0, nh=nh)


def cfg5_dsa(n_keys=65536, batch=8, ih=64, topk=2048, nh=128, shared=False, seed=SEED0 + 5):
    """`batch` independent decode queries; each has its own caches unless shared."""
    g = rng(seed)
    nctx = 1 if shared else batch
    ik = np.empty((nctx, n_keys, IDIM), np.uint8)
    iks = np.empty((nctx, n_keys), np.float32)
    rows = np.empty((nctx, n_keys, KDIM), np.uint8)
    scales = np.empty((nctx, n_keys, NBLK), np.float32)
    for c in range(nctx):
        ik[c], iks[c] = index_keys(g, n_keys)
        rows[c], scales[c] = latent_cache(g, n_keys)
    w = (g.standard_normal((batch, ih), dtype=np.float32) *
         np.float32(1.0 / np.sqrt(float(IDIM * ih)))).astype(np.float32)
    return dict(q_idx=normal_bf16(g, (batch, ih, IDIM)), w=w, ikeys=ik, ikscale=iks,
                q=normal_bf16(g, (batch, nh, KDIM)), rows=rows, scales=scales,
                scale=float(1.0 / np.sqrt(192.0)), n_keys=n_keys, batch=batch, ih=ih,
                topk=topk, nh=nh, shared=shared)
