"""Pins the oracle's scalar casts: known answers + torch's CPU casts (library routines)."""
import json
import os

import numpy as np
import pytest
import torch

KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "kat.json")))


def test_e8m0_known_answers(corc):
    k = KAT["f32_to_e8m0"]
    got = corc.f32_to_e8m0(np.array(k["inputs"], np.float32))
    assert got.tolist() == k["bytes"]
    # torch agrees with the list too (guards the list itself)
    t = torch.tensor(k["inputs"], dtype=torch.float32).to(torch.float8_e8m0fnu).view(torch.uint8)
    assert t.tolist() == k["bytes"]


def test_e2m1_tables(corc):
    for key, nz in (("e2m1_pos_zero", 0), ("e2m1_neg_zero", 1)):
        want = np.array(KAT[key]["values"], np.float32)
        got = np.array([corc.e2m1_value(c, nz) for c in range(16)], np.float32)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), key


def test_e4m3_known_answers(corc):
    cases = KAT["f32_to_e4m3fn"]["cases"]
    x = np.array([c[0] for c in cases], np.float32)
    assert corc.f32_to_e4m3fn(x).tolist() == [c[1] for c in cases]
    nan = KAT["f32_to_e4m3fn_nan"]
    got = corc.f32_to_e4m3fn(np.array(nan["inputs"], np.float32))
    assert all((g & 0x7F) == nan["code_low7"] for g in got.tolist())


def _patterns():
    """A few million fp32 bit patterns: every exponent x a spread of mantissas,
    every 2^12-th pattern, and dense neighbourhoods of the e4m3fn / bf16 rounding edges."""
    rng = np.random.default_rng(0)
    parts = [np.arange(0, 1 << 32, 1 << 12, dtype=np.uint64).astype(np.uint32),
             rng.integers(0, 1 << 32, 1 << 21, dtype=np.uint64).astype(np.uint32)]
    edges = np.array([0.0, 2.0 ** -10, 2.0 ** -9, 2.0 ** -6, 1.0, 1.0625, 240.0, 448.0, 464.0, 480.0,
                      2.0 ** -126, 2.0 ** -127, 3.3e38], np.float32).view(np.uint32)
    for e in edges:
        lo = max(int(e) - 4096, 0)
        r = np.arange(lo, int(e) + 4096, dtype=np.uint64).astype(np.uint32)
        parts += [r, r | np.uint32(0x80000000)]
    return np.unique(np.concatenate(parts))


def _check_against_torch(corc, u):
    f = u.view(np.float32)
    tf = torch.from_numpy(f.copy())
    isnan = np.isnan(f)
    a = corc.f32_to_e4m3fn(f)
    b = tf.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(a[~isnan], b[~isnan])
    assert np.array_equal(a[isnan] & 0x7F, b[isnan] & 0x7F)
    a = corc.f32_to_bf16(f)
    b = tf.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(a[~isnan], b[~isnan])
    a = corc.f32_to_e8m0(f)
    b = tf.to(torch.float8_e8m0fnu).view(torch.uint8).numpy()
    assert np.array_equal(a, b)


def test_casts_match_torch_sampled(corc):
    _check_against_torch(corc, _patterns())


@pytest.mark.exhaustive
def test_casts_match_torch_exhaustive(corc):
    step = 1 << 25
    for start in range(0, 1 << 32, step):
        _check_against_torch(corc, np.arange(start, start + step, dtype=np.uint64).astype(np.uint32))


def test_decoders_match_torch(corc):
    codes = np.arange(256, dtype=np.uint8)
    a = corc.e4m3fn_to_f32(codes)
    b = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    ok = ~np.isnan(b)
    assert np.array_equal(a.view(np.uint32)[ok], b.view(np.uint32)[ok]) and np.isnan(a[~ok]).all()
    a = corc.e8m0_to_f32(codes)
    b = torch.from_numpy(codes).view(torch.float8_e8m0fnu).float().numpy()
    assert np.array_equal(a.view(np.uint32)[:255], b.view(np.uint32)[:255]) and np.isnan(a[255]) and np.isnan(b[255])
