"""Oracle arithmetic of the FlagRot writers (numpy, fp32 with every operation rounded separately).

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Reference followed (file:line in the reference tree):
  fwht                kernels/ref.py:22-33  (= blockflag/hadamard.py:14-26)
  sel_fwht            kernels/ref.py:36-42
  quant_sym4          kernels/ref.py:151-160
  quant_asym_stored   blockflag/formats.py:153-165 (quant_asym_dep), scale words formats.py:135-146,168-174
  quant_asym_error    kernels/codebook_ref.py:100-109 (the error-form dequantisation of kinds asym / asym2)
  static_encode       kernels/ref.py:169-182 (kv_selrot_quant fmt int4), :190-202 (int4a_quant), centring
                      kernels/csrc/attn_decode_v2.cu:1737-1740
  k2_encode           kernels/codebook_ref.py:119-236 with CFG konly / konlya / konlya2 (:62-71)
  head_fwht           integrations/vllm_flagrot/csrc/flagrot_capi.cu:167-201

Division convention.  `true_div=False` (default, the kernel oracle) computes the asymmetric step as
(max - min) * fp32(1/levels), which is what PyTorch does on a GPU device and what the reference's CUDA kernels do
(blockflag/formats.py:155-156, attn_cb_common.cuh:56-58).  `true_div=True` uses IEEE division, which is what the
reference's Python does when it runs on a CPU; it exists so that golden vectors written by the reference on a CPU
pin the structure (operation order, tie rules, flag rules) of this restatement bit for bit.

Parity status
  fwht, quant_sym4, quant_asym_*, scale_word, k2_encode, static quantisers:
      pinned by tests/test_oracle_golden.py against tests/golden/k2_encode_*.npz (written by the reference's
      codebook_ref.encode on a CPU, true_div=True) and by the closed-form checks of tests/test_oracle_quant.py
      (Sylvester matmul, exhaustive scale-word search, brute-force scalar loops, invariants).
  head_fwht: pinned by the fp64 matmul bound (one bf16 rounding) in tests/test_oracle_quant.py.
"""
from __future__ import annotations

import math

import numpy as np

F32 = np.float32
D = 128
RB = 32


# ----------------------------------------------------------------------------------------------- bf16 helpers
def bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit patterns (uint16), round to nearest even."""
    u = np.ascontiguousarray(x, dtype=F32).view(np.uint32).astype(np.uint64)
    r = ((u >> np.uint64(16)) & np.uint64(1)) + np.uint64(0x7FFF)
    return ((u + r) >> np.uint64(16)).astype(np.uint16)


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(F32)


def bf16_round(x: np.ndarray) -> np.ndarray:
    """fp32 values rounded to the bf16 grid (still fp32)."""
    return bf16_to_f32(bf16_bits(x))


def f16_bits(x: np.ndarray) -> np.ndarray:
    return np.asarray(x, dtype=F32).astype(np.float16).view(np.uint16)


def f16_value(bits: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(bits, dtype=np.uint16).view(np.float16).astype(F32)


# ----------------------------------------------------------------------------------------------- transforms
def fwht(x: np.ndarray, n: int) -> np.ndarray:
    """orthonormal Sylvester-Hadamard on every consecutive n-vector of the last axis: butterflies (a+b, a-b) with
    partner distance 1, 2, 4, ... in fp32, then one multiply by fp32(1/sqrt(n))."""
    x = np.asarray(x, dtype=F32)
    y = x.reshape(-1, n).copy()
    lane = np.arange(n)
    h = 1
    while h < n:
        lo = lane[(lane & h) == 0]
        a, b = y[:, lo], y[:, lo + h]
        nxt = np.empty_like(y)
        nxt[:, lo] = a + b
        nxt[:, lo + h] = a - b
        y = nxt
        h *= 2
    return (y * F32(1.0 / math.sqrt(n))).reshape(x.shape)


def sylvester(n: int) -> np.ndarray:
    """orthonormal Sylvester matrix in fp64 (closed form used by the tests)."""
    i = np.arange(n)
    bits = np.bitwise_and(i[:, None], i[None, :])
    par = np.zeros_like(bits)
    while bits.any():
        par ^= bits & 1
        bits >>= 1
    return (1.0 - 2.0 * par) / math.sqrt(n)


def sel_fwht(x: np.ndarray, mask: np.ndarray, rb: int = RB) -> np.ndarray:
    """x fp32 [..., H, Dh]; mask [H, Dh/rb]: rb-vectors with a set flag are replaced by their fwht."""
    m = np.repeat(np.asarray(mask).astype(bool), rb, axis=-1)
    if not m.any():
        return np.asarray(x, dtype=F32)
    return np.where(m, fwht(x, rb), np.asarray(x, dtype=F32))


# ----------------------------------------------------------------------------------------------- quantisers
def _groups(y: np.ndarray) -> np.ndarray:
    y = np.asarray(y, dtype=F32)
    return y.reshape(*y.shape[:-1], y.shape[-1] // RB, RB)


def quant_sym4(y: np.ndarray):
    """symmetric INT4 per 32: s = fp16(amax * fp32(1/7)); q = clamp(rne(y / s), -7, 7), q = 0 where s == 0.
    Returns q int8 [..., Dh], scale words uint16 [..., Dh/32] (fp16 bits), dequantised fp32 [..., Dh]."""
    b = _groups(y)
    amax = np.abs(b).max(-1, keepdims=True)
    sh = (amax * F32(1.0 / 7.0)).astype(np.float16)
    s = sh.astype(F32)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(s != 0, np.rint(b / np.where(s != 0, s, F32(1))), F32(0))
    q = np.clip(q, F32(-7), F32(7)).astype(F32)
    deq = q * s
    return q.astype(np.int8).reshape(y.shape), sh.view(np.uint16)[..., 0], deq.reshape(y.shape)


def scale_word(s: np.ndarray, z: np.ndarray, bits: int = 4) -> np.ndarray:
    """16-bit scale word: the FP16 bit pattern nearest to RN16(s) (distance on the pattern, ties upwards) whose
    `bits` low bits equal z, capped below the infinity pattern."""
    m = 1 << bits
    h = f16_bits(s).astype(np.int32)
    zi = np.asarray(z).astype(np.int32)
    x = np.minimum(np.maximum(h - zi + m // 2, 0) & ~(m - 1), 0x7C00 - m)
    return (x + zi).astype(np.int32)


def _step(mx, mn, lv, true_div):
    rng = mx - mn
    s = rng / F32(lv) if true_div else rng * F32(1.0 / lv)
    return np.maximum(s, F32(1e-12)).astype(F32)


def quant_asym_stored(y: np.ndarray, bits: int = 4, true_div: bool = False):
    """stored form of int4a:32 / int2a:32 (range widened to include 0): codes uint8 [..., Dh] in [0, 2^bits - 1],
    scale words int32 [..., Dh/32] (low `bits` bits = zero point, the word read as FP16 = the scale)."""
    lv = (1 << bits) - 1
    b = _groups(y)
    mn = np.minimum(b.min(-1, keepdims=True), F32(0))
    mx = np.maximum(b.max(-1, keepdims=True), F32(0))
    s = _step(mx, mn, lv, true_div)
    z = np.rint(-mn / s)
    q = np.clip(np.rint(b / s) + z, F32(0), F32(lv))
    return q.astype(np.uint8).reshape(y.shape), scale_word(s, z, bits)[..., 0]


def quant_asym_error(y: np.ndarray, bits: int = 4, true_div: bool = False) -> np.ndarray:
    """dequantisation of int4a:32 / int2a:32 with an FP32 step and an unbounded zero point (the form the selection
    errors of the asymmetric key-only kinds are measured on)."""
    lv = (1 << bits) - 1
    b = _groups(y)
    mn, mx = b.min(-1, keepdims=True), b.max(-1, keepdims=True)
    s = _step(mx, mn, lv, true_div)
    z = np.rint(-mn / s)
    qa = np.clip(np.rint(b / s) + z, F32(0), F32(lv))
    return ((qa - z) * s).astype(F32).reshape(y.shape)


def word_scale(words: np.ndarray) -> np.ndarray:
    """scale magnitude of a stored word: FP16 value of the word without its sign (flag) bit."""
    return f16_value((np.asarray(words).astype(np.int64) & 0x7FFF).astype(np.uint16))


QK_OF_KIND = {"konly": "sym", "konlya": "asym4", "konlya2": "asym2", "int4": "sym", "int4a": "asym4", "int2a": "asym2"}


def quant(y: np.ndarray, qk: str, true_div: bool = False):
    """(stored codes, stored words, dequantisation used by the selection errors) for quantiser qk in
    'sym' (codes int8 in [-7, 7]) | 'asym4' | 'asym2' (codes uint8)."""
    if qk == "sym":
        return quant_sym4(y)
    bits = 4 if qk == "asym4" else 2
    q, w = quant_asym_stored(y, bits, true_div)
    return q, w, quant_asym_error(y, bits, true_div)


def dequant_stored(codes: np.ndarray, words: np.ndarray, qk: str, dtype=np.float64) -> np.ndarray:
    """value of stored codes + words: sym q * s; asym (c - z) * s with z = the low bits of the word."""
    c = _groups(codes.astype(F32)).astype(dtype)
    w = np.asarray(words).astype(np.int64)
    if qk != "sym":
        c = c - (w & (15 if qk == "asym4" else 3))[..., None].astype(dtype)
    return (c * word_scale(w)[..., None].astype(dtype)).reshape(codes.shape)


# ----------------------------------------------------------------------------------------------- static writer
def static_encode(kv_bits: np.ndarray, mask: np.ndarray, fmt: str, kmu: np.ndarray | None = None,
                  true_div: bool = False):
    """kv_bits uint16 [T, 2*Hkv, Dh] (bf16 patterns, K rows first); mask [2*Hkv, Dh/32]; kmu fp32 [Hkv, Dh] or None.
    Returns stored codes [T, 2*Hkv, Dh] and scale words int32 [T, 2*Hkv, Dh/32]."""
    x = bf16_to_f32(kv_bits)
    Hkv = x.shape[1] // 2
    if kmu is not None:
        x = x.copy()
        x[:, :Hkv] = x[:, :Hkv] - np.asarray(kmu, dtype=F32)[None]
    y = sel_fwht(x, mask, RB)
    q, w, _ = quant(y, QK_OF_KIND[fmt], true_div)
    return q, w.astype(np.int32)


def head_fwht(x_bits: np.ndarray, flags: np.ndarray, scale: float) -> np.ndarray:
    """bf16 [T, H, Dh] patterns -> bf16 patterns of scale * (unnormalised +-1 Sylvester) x for flagged heads, a copy
    for the others.  Butterflies in fp32 (partner distance 1, 2, 4, ...), one multiply, one bf16 rounding."""
    x = bf16_to_f32(x_bits)
    n = x.shape[-1]
    y = x.reshape(-1, n).copy()
    lane = np.arange(n)
    h = 1
    while h < n:
        lo = lane[(lane & h) == 0]
        a, b = y[:, lo], y[:, lo + h]
        nxt = np.empty_like(y)
        nxt[:, lo] = a + b
        nxt[:, lo + h] = a - b
        y = nxt
        h *= 2
    y = bf16_bits(y * F32(scale)).reshape(x_bits.shape)
    return np.where(np.asarray(flags).astype(bool)[None, :, None], y, x_bits).astype(np.uint16)


# ----------------------------------------------------------------------------------------------- selecting writer
def tree_sum(p: np.ndarray) -> np.ndarray:
    """halving tree over the last axis: v[:n/2] + v[n/2:] until one element."""
    while p.shape[-1] > 1:
        n = p.shape[-1] // 2
        p = p[..., :n] + p[..., n:]
    return p[..., 0]


def seq_matvec(M: np.ndarray, e: np.ndarray, k0: int, k1: int) -> np.ndarray:
    """u[t, h, i] = M[h, i, k0] * e[t, h, k0] + M[h, i, k0 + 1] * e[t, h, k0 + 1] + ... added left to right, every
    product and sum rounded to fp32."""
    u = M[None, :, :, k0] * e[:, :, None, k0]
    for k in range(k0 + 1, k1):
        u = u + M[None, :, :, k] * e[:, :, None, k]
    return u


def key_local_err(e: np.ndarray, C: np.ndarray) -> np.ndarray:
    """e [T, H, Dh] -> [T, H, Dh/32]: tree(e_a * seq_k(C_jj[a, k] e_k)) per diagonal 32-block j."""
    out = []
    for j in range(e.shape[-1] // RB):
        sl = slice(RB * j, RB * (j + 1))
        ej = e[..., sl]
        out.append(tree_sum(ej * seq_matvec(C[:, sl, sl], ej, 0, RB)))
    return np.stack(out, -1)


def key_head_err(e: np.ndarray, C: np.ndarray) -> np.ndarray:
    """tree(e_i * u_i), u = ((U_0 + U_1) + U_2) + ..., U_b = seq over the columns of 32-block b."""
    nb = e.shape[-1] // RB
    u = seq_matvec(C, e, 0, RB)
    for b in range(1, nb):
        u = u + seq_matvec(C, e, RB * b, RB * (b + 1))
    return tree_sum(e * u)


def k2_encode_keys(x: np.ndarray, C: np.ndarray, qk: str, true_div: bool = False):
    """x fp32 [T, H, Dh] (already centred), C fp32 [H, Dh, Dh] (C_q, not transposed).
    Returns dict(q stored codes, w stored words int32 [T, H, Dh/32] without flag bits, local uint8 [T, H, Dh/32]
    (1 = group stored as H32 x), full bool [T, H] (row stored as H_Dh x), err_local [2, T, H, Dh/32], err_head
    [2, T, H])."""
    x = np.asarray(x, dtype=F32)
    C = np.asarray(C, dtype=F32)
    Dh = x.shape[-1]
    ng = Dh // RB
    qi, wi, di = quant(x, qk, true_div)
    qh, wh, dh = quant(fwht(x, RB), qk, true_div)
    e_i = di - x
    e_h = fwht(dh, RB) - x
    err_l = np.stack([key_local_err(e_i, C), key_local_err(e_h, C)])
    local = err_l[1] < err_l[0]                                       # strict: ties keep the identity
    sel = np.repeat(local, RB, -1)
    q_b = np.where(sel, qh, qi)
    w_b = np.where(local, wh, wi)
    e_b = np.where(sel, e_h, e_i)
    qf, wf, df = quant(fwht(x, Dh), qk, true_div)
    e_f = fwht(df, Dh) - x
    err_h = np.stack([key_head_err(e_b, C), key_head_err(e_f, C)])
    full = err_h[1] < err_h[0]
    q = np.where(full[..., None], qf, q_b)
    w = np.where(full[..., None], wf, w_b).astype(np.int32)
    loc = np.where(full[..., None], np.zeros((1,) * 3, bool), local).astype(np.uint8)
    assert loc.shape[-1] == ng
    return dict(q=q, w=w, local=loc, full=full, err_local=err_l, err_head=err_h)


def k2_encode(kv_bits: np.ndarray, C: np.ndarray, kind: str, kmu: np.ndarray | None = None,
              true_div: bool = False):
    """selecting writer of the key-only 2x2 kinds: kv_bits uint16 [T, 2*Hkv, Dh] bf16 patterns (K rows first).
    Returns (codes [T, 2*Hkv, Dh], words int32 [T, 2*Hkv, Dh/32] WITH flag bits, info dict of the key choice).
    Flags: K word g bit 15 = group g stored as H32 x (only when the row is not stored as H_Dh x); V word 0 bit 15 =
    the token's key row is stored as H_Dh x.  Values: plain group quantisation, no transform."""
    qk = QK_OF_KIND[kind]
    x = bf16_to_f32(kv_bits)
    Hkv = x.shape[1] // 2
    xk = x[:, :Hkv]
    if kmu is not None:
        xk = xk - np.asarray(kmu, dtype=F32)[None]
    kk = k2_encode_keys(xk, C, qk, true_div)
    qv, wv, _ = quant(x[:, Hkv:], qk, true_div)
    wk = kk["w"] | (kk["local"].astype(np.int32) << 15)
    wv = wv.astype(np.int32).copy()
    wv[..., 0] |= kk["full"].astype(np.int32) << 15
    codes = np.concatenate([kk["q"].astype(np.int16), qv.astype(np.int16)], 1)
    return codes, np.concatenate([wk, wv], 1), kk
