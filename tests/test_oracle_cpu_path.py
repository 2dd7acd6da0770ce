"""The torch-CPU restatement of the reference's CPU path (oracle/cpu_path.py, what bench.py times as
the CPU baseline) against the numpy oracle: the two must compute the same thing."""

import math

import numpy as np
import torch

from oracle import attend as oa, cpu_path as cp, kivi as ok, vecinfer as ov


def _kv(shape, seed):
    rng = np.random.default_rng(seed)
    f = np.exp(rng.standard_normal(shape[-1])).astype(np.float32)
    return ((rng.standard_normal(shape).astype(np.float32) * f).astype(np.float16),
            rng.standard_normal(shape).astype(np.float16))


def test_kivi_round_trip_is_the_oracle_bit_for_bit():
    k, v = _kv((1, 2, 75, 64), 1)           # ragged last group
    for x, axis in ((k, -2), (v, -1)):
        for bits, g in ((4, 32), (2, 16), (8, 32)):
            got = cp.kivi_round_trip(torch.from_numpy(x), axis, g, (1 << bits) - 1).numpy()
            want = ok.quant_dequant_along(x, axis, g, (1 << bits) - 1)
            assert got.dtype == np.float16 and np.array_equal(got, want)


def test_quantize_vq_agrees_with_the_oracle_off_ties():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((2, 40, 32)).astype(np.float16)
    cb = rng.standard_normal((64, 8)).astype(np.float16)
    got = cp.quantize_vq(torch.from_numpy(x), torch.from_numpy(cb), 8).numpy()
    want = ov.quantize_vq(x, cb, 8)
    assert got.shape == want.shape == (2, 40, 4)
    assert np.array_equal(got, want)        # random data: no two centroids at equal distance


def test_decode_dequant_then_sdpa_is_the_reference_attend():
    rng = np.random.default_rng(3)
    B, Hq, Hkv, S, D, g = 1, 8, 2, 96, 64, 32
    kf, vf = _kv((B, Hkv, S, D), 4)
    kq = ok.group_quant_codes(kf, -2, g, 15)
    vq = ok.group_quant_codes(vf, -1, g, 15)
    q = rng.standard_normal((B, Hq, 1, D)).astype(np.float16)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a))
    got = cp.decode_dequant_then_sdpa(t(q), *[t(a) for a in kq], *[t(a) for a in vq], g, 0.125).float().numpy()
    want = oa.reference_attend(q, *kq, *vq, g, 0.125)
    # the reference's dequantise-then-SDPA arm rounds K_hat / V_hat to fp16 first
    assert np.max(np.abs(got - want)) < 5e-3


def test_chunked_prefill_matches_the_oracle():
    B, Hq, Hkv, D, g, R, bits, chunk = 1, 4, 2, 64, 16, 32, 4, 24
    k, v = _kv((B, Hkv, 40 + 3 * chunk, D), 5)
    q = np.random.default_rng(6).standard_normal((B, Hq, 3 * chunk, D)).astype(np.float16)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a))
    outs = cp.chunked_prefill([t(q[:, :, i * chunk:(i + 1) * chunk]) for i in range(3)],
                              [t(k[:, :, 40 + i * chunk:40 + (i + 1) * chunk]) for i in range(3)],
                              [t(v[:, :, 40 + i * chunk:40 + (i + 1) * chunk]) for i in range(3)],
                              t(k[:, :, :40]), t(v[:, :, :40]), bits, g, R, 1 / math.sqrt(D))
    got = torch.cat(outs, dim=2).float().numpy()
    want = oa.chunked_prefill(q, k[:, :, 40:], v[:, :, 40:], chunk, bits, g, R, 1 / math.sqrt(D),
                              prefix_k=k[:, :, :40], prefix_v=v[:, :, :40])
    assert np.max(np.abs(got - want)) < 2e-3
