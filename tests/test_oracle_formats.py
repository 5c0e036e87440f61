"""Pins the oracle's scalar formats (bf16, OCP e4m3fn) against torch's casts,
which are the library routines for those formats."""
import numpy as np
import torch


def _torch_bf16_bits(x):
    return torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def _torch_e4m3(x):
    return torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def test_bf16_rne_matches_torch(oracle):
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 10,
        # exact ties: bf16 value + half an ulp
        (np.arange(1, 4000, dtype=np.uint32) << 16 | 0x8000).view(np.float32) ,
        ((np.arange(1, 4000, dtype=np.uint32) + 0x3f00) << 16 | 0x8000).view(np.float32),
        np.array([0.0, -0.0, 1e-40, -1e-40, 3.3895e38, np.inf, -np.inf], np.float32),
    ])
    want = _torch_bf16_bits(x)
    assert np.array_equal(oracle.np_f32_to_bf16_bits(x), want)
    sub = np.r_[0:2000, 20000:21000, len(x) - 7:len(x)]
    assert np.array_equal(oracle.c_f32_to_bf16_bits(x[sub]), want[sub])
    assert np.array_equal(oracle.np_bf16_bits_to_f32(want).view(np.uint32),
                          torch.from_numpy(want.view(np.int16)).view(torch.bfloat16).float().numpy().view(np.uint32))


def test_e4m3fn_decode_table_matches_torch(oracle):
    want = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    for got in (oracle.np_e4m3fn_table(), oracle.c_e4m3fn_table()):
        assert np.array_equal(np.isnan(got), np.isnan(want))
        ok = ~np.isnan(want)
        assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
    assert want[0x7E] == 448.0 and want[0x01] == 2.0 ** -9


def test_e4m3fn_encode_matches_torch_on_codes_midpoints_and_sweep(oracle):
    tab = oracle.np_e4m3fn_table()
    pos = tab[:127].astype(np.float64)
    mids = (pos[:-1] + pos[1:]) / 2  # every tie point, exactly representable in fp32
    rng = np.random.default_rng(2)
    cases = np.concatenate([
        pos, -pos, mids, -mids,
        np.nextafter(mids.astype(np.float32), np.float32(np.inf)),
        np.nextafter(mids.astype(np.float32), np.float32(-np.inf)),
        rng.uniform(-448, 448, 50000), rng.standard_normal(50000) * 0.01,
        rng.standard_normal(50000) * 2.0 ** -8, np.array([448.0, -448.0, 0.0, -0.0]),
    ]).astype(np.float32)
    want = _torch_e4m3(cases)
    got_np = oracle.np_f32_to_e4m3fn(cases)
    # -0.0 encodes as 0x80 in both
    assert np.array_equal(got_np, want)
    sub = np.r_[0:len(pos) * 2 + len(mids) * 4, len(cases) - 4000:len(cases)]
    assert np.array_equal(oracle.c_f32_to_e4m3fn(cases[sub]), want[sub])


def test_e4m3fn_saturates_past_448(oracle):
    x = np.array([449.0, 463.9, 464.0, 1e4, -1e4, 3e38], np.float32)
    for f in (oracle.np_f32_to_e4m3fn, oracle.c_f32_to_e4m3fn):
        got = f(x)
        assert list(got & 0x7F) == [0x7E] * 6
