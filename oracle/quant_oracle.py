"""TEST INFRASTRUCTURE ONLY - CPU restatement (numpy) of the block quantisers in front of the GEMM.

Nothing in the product path imports this file: only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may, and only as the checker.

The reference has no quantiser: its operands arrive quantised from the un-vendored harness
(1-amd-fp8-mm/0-amd-fp8-mm-new-begins.py:66-77 states what arrives: e4m3 a [M,K] and b [N,K] stored
K-major, fp32 a_scale [M,K/128] per 1x128 block, b_scale [N/128,K/128] per 128x128 block).  The rule
restated here is the one this build defines for its inputs and its HIP quantisers:

    scale = max(max|x| over the block / 448, 1e-12)           fp32 arithmetic
    q     = e4m3fn( clamp(x / scale, -448, 448) )              fp32 division, round to nearest even

Outputs are returned in STORAGE order (what the C ABI writes):  q[K][rows] uint8 codes,
scale[K/128][rows] (activations) or scale[K/128][ceil(rows/128)] (weights)
(storage order of 1-amd-fp8-mm/amd-fp8-mm-submission.py:66-75).

How each function is pinned (tests/test_quant_oracle.py):
  * encode_e4m3fn   against torch's own float32 -> float8_e4m3fn cast (a library routine of the
                    container's torch) on every representable value, every rounding midpoint, their
                    fp32 neighbours on both sides, subnormals, +-0 and two million random values;
                    decode(encode(v)) == v for all 254 finite codes; ties go to the even code
  * quantize_a_ref / quantize_b_ref
                    bit-exact agreement with an independent torch implementation (torch's cast and
                    torch's amax/div) on random data with outliers, all-zero blocks and row tails;
                    invariants: |decoded q| <= 448, the largest |x| of every non-zero block maps to
                    code 448, relative error of normal values <= 2^-4, re-quantising the dequantised
                    values returns the same codes
  * gather_a_ref    defined by the identity it is checked against: gather_a_ref(quantize_a_ref(x), map) must
                    equal quantize_a_ref(x, map) bit for bit (a block's scale and bytes depend on its own row
                    only), including out-of-range entries; plus a hand-written 3-row case
  * fnuz_to_fn_ref  (e4m3fnuz, the reference's gfx942 type, 1-amd-fp8-mm/amd-fp8-mm-submission.py:20-21:
                    bias 8, NaN 0x80, no -0)  torch's own float8_e4m3fnuz -> float32 -> float8_e4m3fn
                    casts on all 256 codes
"""
import numpy as np

BLOCK = 128
FP8_MAX = np.float32(448.0)
TINY = np.float32(1e-12)


def _positive_values() -> np.ndarray:
    """float64[127]: the non-negative finite e4m3fn values, code 0x00..0x7E, closed form."""
    v = np.empty(127, dtype=np.float64)
    for code in range(127):
        e, m = code >> 3, code & 7
        v[code] = m * 2.0 ** -9 if e == 0 else (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return v


_VALS = _positive_values()
_MIDS = (_VALS[:-1] + _VALS[1:]) / 2.0          # exact in float64


def encode_e4m3fn(x: np.ndarray) -> np.ndarray:
    """float32 array with |x| <= 448 (or NaN) -> uint8 e4m3fn codes, round to nearest, ties to even.

    NaN maps to 0x7F with the sign bit of the input.  Values beyond 448 are the caller's to clamp.
    """
    x = np.asarray(x, dtype=np.float32)
    ax = np.abs(x).astype(np.float64)
    nan = np.isnan(ax)
    ax = np.where(nan, 0.0, ax)
    code = np.searchsorted(_MIDS, ax, side="left")          # first midpoint >= |x|  ->  |x| <= mids[code]
    # |x| exactly on a midpoint between code and code+1: take the even one
    on_mid = (code < 126) & (ax == _MIDS[np.minimum(code, 125)])
    code = np.where(on_mid & (code % 2 == 1), code + 1, code)
    code = np.where(nan, 0x7F, code).astype(np.uint8)
    sign = (np.signbit(x).astype(np.uint8)) << 7
    return code | sign


def quantize_a_ref(x: np.ndarray, row_map=None):
    """x float32 [T, K] -> (q uint8 [K][M], scale float32 [K/128][M]); one scale per row and K block.

    With ``row_map`` (int [M]) output row i comes from input row row_map[i] (out-of-range: zero row).
    """
    x = np.asarray(x, dtype=np.float32)
    if row_map is not None:
        row_map = np.asarray(row_map, dtype=np.int64)
        ok = (row_map >= 0) & (row_map < x.shape[0])
        g = np.zeros((row_map.size, x.shape[1]), dtype=np.float32)
        g[ok] = x[row_map[ok]]
        x = g
    m, k = x.shape
    assert k % BLOCK == 0
    xb = x.reshape(m, k // BLOCK, BLOCK)
    amax = np.abs(xb).max(axis=2)
    scale = np.maximum(amax / FP8_MAX, TINY).astype(np.float32)
    q = np.clip(xb / scale[:, :, None], -FP8_MAX, FP8_MAX).astype(np.float32)
    codes = encode_e4m3fn(q.reshape(m, k))
    return np.ascontiguousarray(codes.T), np.ascontiguousarray(scale.T)


def gather_a_ref(q: np.ndarray, scale: np.ndarray, row_map) -> tuple:
    """Storage-order q uint8 [K][T], scale float32 [K/128][T] -> the same for rows row_map (int [M]).

    Entries of row_map outside [0, T) give zero bytes and the scale 1e-12 (a zero row quantised).
    Row copy into expert order: 2-amd-moe/3-amd-fp8-moe-hip-myhgemm.py:174-191.
    """
    q = np.asarray(q, dtype=np.uint8)
    scale = np.asarray(scale, dtype=np.float32)
    row_map = np.asarray(row_map, dtype=np.int64)
    ok = (row_map >= 0) & (row_map < q.shape[1])
    safe = np.where(ok, row_map, 0)
    if q.shape[1] == 0:
        return np.zeros((q.shape[0], row_map.size), np.uint8), np.full((scale.shape[0], row_map.size), TINY, np.float32)
    out_q = np.where(ok[None, :], q[:, safe], np.uint8(0)).astype(np.uint8)
    out_s = np.where(ok[None, :], scale[:, safe], TINY).astype(np.float32)
    return np.ascontiguousarray(out_q), np.ascontiguousarray(out_s)


def quantize_b_ref(w: np.ndarray):
    """w float32 [N, K] -> (q uint8 [K][N], scale float32 [K/128][ceil(N/128)]); one scale per 128x128 block."""
    w = np.asarray(w, dtype=np.float32)
    n, k = w.shape
    assert k % BLOCK == 0
    nb, kb = (n + BLOCK - 1) // BLOCK, k // BLOCK
    wp = np.zeros((nb * BLOCK, k), dtype=np.float32)
    wp[:n] = w
    wb = wp.reshape(nb, BLOCK, kb, BLOCK)
    amax = np.abs(wb).max(axis=(1, 3))
    scale = np.maximum(amax / FP8_MAX, TINY).astype(np.float32)                 # [nb, kb]
    q = np.clip(wb / scale[:, None, :, None], -FP8_MAX, FP8_MAX).astype(np.float32)
    codes = encode_e4m3fn(q.reshape(nb * BLOCK, k)[:n])
    return np.ascontiguousarray(codes.T), np.ascontiguousarray(scale.T)


def decode_e4m3fnuz(codes: np.ndarray) -> np.ndarray:
    """uint8 e4m3fnuz codes -> float32: (-1)^s 2^(e-8) (1 + m/8), subnormals m 2^-10, 0x80 = NaN, no -0."""
    c = np.asarray(codes, dtype=np.uint8).astype(np.int32)
    e, m = (c >> 3) & 15, c & 7
    mag = np.where(e == 0, m * 2.0 ** -10, (1.0 + m / 8.0) * np.exp2(e.astype(np.float64) - 8))
    v = np.where(c & 0x80, -mag, mag)
    return np.where(c == 0x80, np.nan, v).astype(np.float32)


def fnuz_to_fn_ref(codes: np.ndarray) -> np.ndarray:
    """e4m3fnuz codes -> e4m3fn codes of the same value (round to nearest even where fn is coarser)."""
    out = encode_e4m3fn(decode_e4m3fnuz(codes))
    return np.where(np.asarray(codes, dtype=np.uint8) == 0x80, np.uint8(0x7F), out).astype(np.uint8)
