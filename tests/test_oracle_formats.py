"""CPU: the oracle's number-format tables against every independent statement of them
(committed golden file from torch's fp8 views / the OCP definitions, the reference test's
bit-level emulation, the restated interpreter up-cast)."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import formats

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "formats.json")))


def _bits(x):
    return np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_fp8_table_matches_golden_bitwise(fmt):
    tab = formats.fp8_table(fmt)
    gold = np.array(GOLD[fmt], dtype=np.uint32).view(np.float32)
    fin = ~np.isnan(gold)
    assert np.array_equal(np.isnan(tab), np.isnan(gold))
    assert np.array_equal(_bits(tab)[fin], _bits(gold)[fin])


@pytest.mark.parametrize("fmt,tdt", [("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)])
def test_fp8_table_matches_torch_view(fmt, tdt):
    # precedent: the reference builds fp8 test inputs through torch views (test_core.py:3041-3046)
    ref = torch.arange(256, dtype=torch.uint8).view(tdt).float().numpy()
    tab = formats.fp8_table(fmt)
    fin = ~np.isnan(ref)
    assert np.array_equal(_bits(tab)[fin], _bits(ref)[fin]) and np.array_equal(np.isnan(tab), ~fin)


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_fp8_table_matches_reference_emulation(fmt):
    # test_conversions.py:178-209 algorithm, valid up to max_repr (:295-303)
    eb, mb, bias, max_code = formats.FP8_FORMATS[fmt]
    codes = np.concatenate([np.arange(0, max_code + 1), np.arange(128, 128 + max_code + 1)])
    assert np.array_equal(_bits(formats.fp8_upcast_emulated(codes, fmt)), _bits(formats.fp8_table(fmt)[codes]))


def test_format_constants():
    # max finite values: test_conversions.py:312-314 (0x47600000 = 57344, 0x43e00000 = 448)
    assert formats.fp8_table("e4m3")[0x7E] == 448.0 and formats.fp8_table("e5m2")[0x7B] == 57344.0
    assert np.float32(448.0).view(np.uint32) == 0x43E00000 and np.float32(57344.0).view(np.uint32) == 0x47600000
    assert formats.fp8_table("e4m3")[1] == 2.0 ** -9 and formats.fp8_table("e5m2")[1] == 2.0 ** -16
    assert np.isnan(formats.fp8_table("e4m3")[0x7F]) and np.isinf(formats.fp8_table("e5m2")[0x7C])


def test_interpreter_upcast_restatement():
    # agrees with the closed form on all finite e4m3 codes and all NORMAL e5m2 codes; its two
    # quirks (e4m3 NaN -> 480, e5m2 subnormals mangled) are documented and not adopted
    c = np.arange(256)
    t4 = formats.fp8_table("e4m3")
    h4 = formats.fp8_upcast_interpreter(c, "e4m3").view(np.float16).astype(np.float32)
    fin = ~np.isnan(t4)
    assert np.array_equal(_bits(h4)[fin], _bits(t4)[fin])
    assert h4[0x7F] == 480.0
    t5 = formats.fp8_table("e5m2")
    h5 = formats.fp8_upcast_interpreter(c, "e5m2").view(np.float16).astype(np.float32)
    normal = np.isfinite(t5) & (((c >> 2) & 31) != 0)
    assert np.array_equal(_bits(h5)[normal], _bits(t5)[normal])
    sub = (((c >> 2) & 31) == 0) & ((c & 3) != 0)
    assert np.all(h5[sub] != t5[sub])   # the quirk: e5m2 subnormals lose their value


def test_mx_tables_match_golden():
    assert np.array_equal(_bits(formats.e2m1_table()), np.array(GOLD["e2m1"], dtype=np.uint32))
    e8 = formats.e8m0_table()
    g8 = np.array(GOLD["e8m0"], dtype=np.uint32)
    assert np.array_equal(_bits(e8)[:255], g8[:255]) and np.isnan(e8[255])
    # closed form: consecutive scales differ by exactly 2, 127 is 1.0
    assert e8[127] == 1.0 and np.all(e8[1:255] / e8[0:254] == 2.0)


def test_mx_tables_match_torch_views_when_available():
    if hasattr(torch, "float8_e8m0fnu"):
        ref = torch.arange(255, dtype=torch.uint8).view(torch.float8_e8m0fnu).float().numpy()
        assert np.array_equal(_bits(formats.e8m0_table())[:255], _bits(ref))
    else:
        pytest.skip("torch has no e8m0 dtype")


def test_fp4_pack_roundtrip_low_nibble_first():
    codes = np.arange(16, dtype=np.uint8).reshape(1, 16)
    packed = formats.pack_fp4(codes)
    assert packed[0, 0] == 0x10 and packed[0, 7] == 0xFE  # element 2i low, 2i+1 high
    assert np.array_equal(formats.unpack_fp4(packed), codes)


@pytest.mark.parametrize("fmt,tdt", [("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)])
def test_encode_fp8_is_rtne_inverse(fmt, tdt):
    tab = formats.fp8_table(fmt)
    fin = np.isfinite(tab)
    c = np.arange(256)[fin]
    c = c[c != 0x80]  # -0 encodes to itself via signbit; keep it separate
    assert np.array_equal(formats.encode_fp8(tab[c], fmt), c.astype(np.uint8))
    rng = np.random.default_rng(0)
    lim = 448 if fmt == "e4m3" else 57344
    x = (rng.standard_normal(20000) * lim / 4).astype(np.float32)
    x = x[np.abs(x) < lim]
    assert np.array_equal(formats.encode_fp8(x, fmt), torch.from_numpy(x).to(tdt).view(torch.uint8).numpy())
    assert formats.encode_fp8(np.array([1e9], dtype=np.float32), fmt)[0] == formats.FP8_FORMATS[fmt][3]


def test_round_bf16_matches_torch_incl_ties():
    x = np.concatenate([np.random.default_rng(1).standard_normal(5000).astype(np.float32),
                        (1.0 + np.arange(64) * 2.0 ** -8).astype(np.float32)])  # exact ties
    assert np.array_equal(_bits(formats.round_bf16(x)), _bits(torch.from_numpy(x).bfloat16().float().numpy()))
