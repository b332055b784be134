"""Pins oracle/quant_oracle.py (the CPU restatement of the block quantisers) without the reference,
which has no quantiser: against torch's own e4m3fn cast, an independent torch implementation of the
rule, and the invariants the rule implies."""
import importlib

import numpy as np
import pytest
import torch


@pytest.fixture(scope="module")
def qo():
    return importlib.import_module("oracle.quant_oracle")


def _torch_codes(x: np.ndarray) -> np.ndarray:
    return torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def test_encode_matches_torch_cast_on_critical_values(qo, oracle):
    table = oracle.e4m3fn_table().astype(np.float64)
    pos = np.sort(table[:127])
    mids = (pos[:-1] + pos[1:]) / 2
    crit = np.concatenate([pos, mids]).astype(np.float32)
    crit = np.concatenate([crit, np.nextafter(crit, np.float32(np.inf)), np.nextafter(crit, np.float32(-np.inf))])
    crit = crit[(crit >= 0) & (crit <= 448)]
    crit = np.concatenate([crit, -crit, np.array([0.0, -0.0, 1e-30, -1e-30, 2.0 ** -10, 2.0 ** -11], dtype=np.float32)])
    assert np.array_equal(qo.encode_e4m3fn(crit), _torch_codes(crit))


def test_encode_matches_torch_cast_on_random_values(qo):
    rng = np.random.default_rng(7)
    x = np.concatenate([
        rng.uniform(-448, 448, 1_000_000),
        rng.standard_normal(500_000) * 0.05,            # subnormal range of e4m3fn
        np.ldexp(rng.uniform(1, 2, 500_000), rng.integers(-12, 9, 500_000)) * rng.choice([-1, 1], 500_000),
    ]).astype(np.float32)
    x = np.clip(x, -448, 448)
    assert np.array_equal(qo.encode_e4m3fn(x), _torch_codes(x))


def test_encode_decode_round_trip_and_ties_to_even(qo, oracle):
    table = oracle.e4m3fn_table()
    finite = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    assert np.array_equal(qo.encode_e4m3fn(table[finite]), finite)
    # the midpoint of codes c, c+1 goes to the even one
    pos = table[:127].astype(np.float64)
    mids = ((pos[:-1] + pos[1:]) / 2).astype(np.float32)
    got = qo.encode_e4m3fn(mids)
    want = np.array([c if c % 2 == 0 else c + 1 for c in range(126)], dtype=np.uint8)
    assert np.array_equal(got, want)
    nan = qo.encode_e4m3fn(np.array([np.nan], dtype=np.float32))
    assert (nan[0] & 0x7F) == 0x7F


def _draw(rng, rows, k):
    x = rng.standard_normal((rows, k)).astype(np.float32)
    x[rng.random((rows, k)) < 0.01] *= 20
    x[1, :128] = 0                                    # an all-zero block
    x[2, 128:256] *= 1e-20                            # a block far below the smallest scale
    return x


def test_quantize_a_agrees_with_independent_torch_rule(qo, pkg):
    rng = np.random.default_rng(11)
    x = _draw(rng, 130, 384)
    q, s = qo.quantize_a_ref(x)
    ta, ts = pkg.inputs.quantize_a(torch.from_numpy(x))
    assert np.array_equal(q, ta.t().contiguous().view(torch.uint8).numpy())
    assert np.array_equal(s, ts.t().contiguous().numpy())
    assert q.shape == (384, 130) and s.shape == (3, 130)


def test_quantize_b_agrees_with_independent_torch_rule(qo, pkg):
    rng = np.random.default_rng(12)
    w = _draw(rng, 200, 256) * 0.02                   # 200 rows: the second 128-row block is partial
    q, s = qo.quantize_b_ref(w)
    tb, ts = pkg.inputs.quantize_b(torch.from_numpy(w))
    assert np.array_equal(q, tb.t().contiguous().view(torch.uint8).numpy())
    assert np.array_equal(s, ts.t().contiguous().numpy())
    assert q.shape == (256, 200) and s.shape == (2, 2)


def test_quantizer_invariants(qo, oracle):
    rng = np.random.default_rng(13)
    x = _draw(rng, 64, 512)
    q, s = qo.quantize_a_ref(x)
    table = oracle.e4m3fn_table()
    dq = table[q]                                       # [K][M]
    assert np.all(np.abs(dq) <= 448)
    xb = x.reshape(64, 4, 128)
    amax = np.abs(xb).max(axis=2)                       # [M][KB]
    dqb = np.abs(dq.T.reshape(64, 4, 128)).max(axis=2)
    assert np.array_equal(dqb[amax > 1e-9], np.full((amax > 1e-9).sum(), 448, dtype=np.float32))
    # relative error of values that land on normal codes: half an e4m3 ulp = 2^-4
    deq = dq.T.reshape(64, 4, 128) * s.T[:, :, None]
    normal = np.abs(dq.T.reshape(64, 4, 128)) >= 2.0 ** -6
    rel = np.abs(deq - xb)[normal] / np.abs(xb)[normal]
    assert rel.max() <= 2.0 ** -4 * (1 + 1e-6)
    # re-quantising the dequantised values returns the same codes
    q2, _ = qo.quantize_a_ref(deq.reshape(64, 512).astype(np.float32))
    assert np.array_equal(q2, q)


def test_row_map_gathers_rows(qo):
    rng = np.random.default_rng(14)
    x = rng.standard_normal((10, 128)).astype(np.float32)
    row_map = np.array([3, 3, 0, 9, -1, 10, 5])
    q, s = qo.quantize_a_ref(x, row_map)
    qf, sf = qo.quantize_a_ref(x)
    for i, r in enumerate(row_map):
        if 0 <= r < 10:
            assert np.array_equal(q[:, i], qf[:, r]) and s[0, i] == sf[0, r]
        else:
            assert not q[:, i].any() and s[0, i] == np.float32(1e-12)


def test_gather_of_quantised_rows_equals_quantising_gathered_rows(qo):
    rng = np.random.default_rng(15)
    x = (rng.standard_normal((37, 384)) * rng.choice([1e-3, 1.0, 50.0], size=(37, 1))).astype(np.float32)
    x[5] = 0
    row_map = np.concatenate([rng.integers(0, 37, size=90), [-1, 37, 1000, -5, 0, 36]])
    rng.shuffle(row_map)
    want_q, want_s = qo.quantize_a_ref(x, row_map)
    got_q, got_s = qo.gather_a_ref(*qo.quantize_a_ref(x), row_map)
    assert got_q.shape == want_q.shape == (384, 96) and got_s.shape == want_s.shape == (3, 96)
    assert np.array_equal(got_q, want_q) and np.array_equal(got_s, want_s)
    # by hand: three rows, one K block
    q = np.arange(3 * 128, dtype=np.uint8).reshape(128, 3)
    sc = np.array([[0.5, 2.0, 8.0]], dtype=np.float32)
    gq, gs = qo.gather_a_ref(q, sc, [2, 0, 3, 2])
    assert np.array_equal(gq[:, 0], q[:, 2]) and np.array_equal(gq[:, 1], q[:, 0]) and not gq[:, 2].any() and np.array_equal(gq[:, 3], q[:, 2])
    assert gs.tolist() == [[8.0, 0.5, float(np.float32(1e-12)), 8.0]]
    # no source rows at all: every entry is out of range
    eq, es = qo.gather_a_ref(np.zeros((128, 0), np.uint8), np.zeros((1, 0), np.float32), [0, 1])
    assert eq.shape == (128, 2) and not eq.any() and (es == np.float32(1e-12)).all()


def test_fnuz_to_fn_against_torch_casts(qo):
    codes = np.arange(256, dtype=np.uint8)
    vals = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fnuz).float()
    assert np.array_equal(np.nan_to_num(qo.decode_e4m3fnuz(codes), nan=-777.0), np.nan_to_num(vals.numpy(), nan=-777.0))
    want = vals.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = qo.fnuz_to_fn_ref(codes)
    finite = codes != 0x80
    assert np.array_equal(got[finite], want[finite])
    assert got[0x80] == 0x7F                                   # the fnuz NaN becomes an fn NaN
    # exact wherever the magnitude code is >= 16
    exact = finite & ((codes & 0x7F) >= 16)
    tab = np.array([(((c & 0x7F) - 8) & 0x7F) | (c & 0x80) for c in range(256)], dtype=np.uint8)
    assert np.array_equal(got[exact], tab[exact])
