"""CPU tests of the packed-tensor container and file format: the documented byte layout decoded by hand must
reproduce the oracle's de-quantized tensor, files round-trip, layout conversions are permutations."""
import json

import numpy as np
import pytest
import torch

from quartet_amd import packed as P
from tests.util import make_input, to_oracle

E2M1 = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])


def decode_by_the_book(p):
    """Values from bytes, following the format description literally (row-major codes)."""
    codes = p.codes.to(torch.int64)
    nib = torch.stack((codes & 15, codes >> 4), dim=-1).view(p.rows, p.cols)          # low nibble = even element
    mag = E2M1[nib & 7]
    val = torch.where((nib & 8) != 0, -mag, mag)
    scale = torch.pow(2.0, (p.scales.to(torch.float64) - 127)).float() * np.float32(p.post_scale)
    return val * scale.repeat_interleave(32, dim=1)


def oracle_packed(oracle, x, mode, kind, signs=None):
    q = oracle.quantize(to_oracle(x), 32, signs=None if signs is None else signs.numpy(), mode=mode, want_mask=(kind == "quest"),
                        want_dequant=True)
    mask = torch.from_numpy(q["mask"]) if q["mask"] is not None else None
    sb = 0 if signs is None else sum(1 << j for j in range(32) if signs[j] < 0)
    p = P.PackedTensor(torch.from_numpy(q["codes"]), torch.from_numpy(q["scales"]), mask, x.shape[0], x.shape[1], "rowmajor", 32,
                       sb, kind)
    return p, q


@pytest.mark.parametrize("kind", ["quest", "absmax"])
def test_documented_layout_decodes_to_the_oracle_tensor(oracle, kind):
    x = make_input(48, 256, torch.float32, seed=5)
    signs = torch.randint(0, 2, (32,), generator=torch.Generator().manual_seed(2)) * 2 - 1
    p, q = oracle_packed(oracle, x, oracle.QUEST_RTN if kind == "quest" else oracle.ABSMAX_RTN, kind, signs)
    want = torch.from_numpy(q["dequant"].astype(np.float32))
    got = decode_by_the_book(p)
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))
    if kind == "quest":
        bits = np.unpackbits(q["mask"], axis=1, bitorder="little").astype(bool)
        assert np.array_equal(p.clip_mask().numpy(), bits)
    else:
        assert p.clip_mask() is None and p.post_scale == float(np.float32(1.0 / 0.75))


def test_file_round_trip(oracle, tmp_path):
    xa = make_input(32, 128, torch.bfloat16, seed=1)
    xb = make_input(16, 64, torch.bfloat16, seed=2)
    pa, _ = oracle_packed(oracle, xa, oracle.QUEST_RTN, "quest")
    pb, _ = oracle_packed(oracle, xb, oracle.ABSMAX_RTN, "absmax")
    pa = P.PackedTensor(pa.codes, pa.scales, pa.maskbits, 32, 128, "rowmajor", 32, 0x8000_0001, "quest").to_layout("tiled")
    path = tmp_path / "acts.safetensors"
    P.save_packed(path, {"layer0.x": pa, "layer0.e": pb}, extra_metadata={"step": "7"})
    back = P.load_packed(path)
    assert set(back) == {"layer0.x", "layer0.e"}
    for name, want in (("layer0.x", pa), ("layer0.e", pb)):
        got = back[name]
        assert torch.equal(got.codes, want.codes) and torch.equal(got.scales, want.scales)
        assert (got.maskbits is None) == (want.maskbits is None)
        if want.maskbits is not None:
            assert torch.equal(got.maskbits, want.maskbits)
        assert (got.rows, got.cols, got.layout, got.hadamard_dim, got.sign_bits, got.scale_kind) == \
               (want.rows, want.cols, want.layout, want.hadamard_dim, want.sign_bits, want.scale_kind)
    from safetensors import safe_open
    with safe_open(str(path), framework="pt") as f:
        meta = f.metadata()
        assert meta["step"] == "7"
        assert json.loads(meta["quartet_mxfp4"])["version"] == P.FORMAT_VERSION
        assert set(f.keys()) == {"layer0.x.e2m1", "layer0.x.e8m0", "layer0.x.mask", "layer0.e.e2m1", "layer0.e.e8m0"}


def test_reader_rejects_foreign_and_newer_files(tmp_path):
    from safetensors.torch import save_file
    plain = tmp_path / "plain.safetensors"
    save_file({"w": torch.zeros(4)}, str(plain))
    with pytest.raises(ValueError, match="not a packed-tensor file"):
        P.load_packed(plain)
    newer = tmp_path / "newer.safetensors"
    save_file({"w": torch.zeros(4)}, str(newer), metadata={"quartet_mxfp4": json.dumps({"version": 99, "tensors": {}})})
    with pytest.raises(ValueError, match="version 99"):
        P.load_packed(newer)
    p = P.PackedTensor(torch.zeros(16, 64, dtype=torch.uint8), torch.zeros(16, 4, dtype=torch.uint8), None, 16, 128)
    with pytest.raises(ValueError, match="collides"):
        P.save_packed(tmp_path / "x.safetensors", {"a.e2m1": p})


def test_tiled_layout_is_the_documented_permutation():
    R, C = 48, 384
    codes = torch.arange(R * C // 2, dtype=torch.int64).remainder(251).to(torch.uint8).view(R, C // 2)
    p = P.PackedTensor(codes, torch.zeros(R, C // 32, dtype=torch.uint8), None, R, C)
    t = p.to_layout("tiled")
    assert t.layout == "tiled" and t.to_layout("tiled") is t
    flat = t.codes.flatten()
    for r, kb, b in ((0, 0, 0), (17, 2, 5), (47, 2, 63), (16, 0, 0), (33, 1, 40)):
        off = ((r // 16) * (C // 128) + kb) * 1024 + (r % 16) * 64 + b   # [R/16][C/128][16 rows][64 bytes]
        assert flat[off] == codes[r, kb * 64 + b]
    assert torch.equal(t.to_layout("rowmajor").codes, codes)
    with pytest.raises(ValueError):
        P.PackedTensor(codes[:40], torch.zeros(40, C // 32, dtype=torch.uint8), None, 40, C).to_layout("tiled")


@pytest.mark.parametrize("R,G", [(128, 4), (32, 1), (130, 5), (256, 8), (384, 12)])
def test_blocked_scale_order(R, G):
    s = torch.randint(0, 256, (R, G), generator=torch.Generator().manual_seed(R + G), dtype=torch.uint8)
    blocked = P.scales_to_blocked(s)
    rb, gb = -(-R // 128), -(-G // 4)
    assert blocked.shape == (rb * gb * 512,)
    for r, g in ((0, 0), (R - 1, G - 1), (R // 2, G // 2), (min(R - 1, 37), 0)):
        block = (r // 128) * gb + g // 4
        rr, gg = r % 128, g % 4
        assert blocked[block * 512 + (rr % 32) * 16 + (rr // 32) * 4 + gg] == s[r, g]
    assert torch.equal(P.scales_from_blocked(blocked, R, G), s)
    with pytest.raises(ValueError):
        P.scales_from_blocked(blocked[:-1], R, G)


def test_container_validation():
    u8 = lambda *shape: torch.zeros(*shape, dtype=torch.uint8)
    P.PackedTensor(u8(4, 16), u8(4, 1), u8(4, 4), 4, 32)
    with pytest.raises(ValueError):
        P.PackedTensor(u8(4, 16), u8(4, 1), None, 4, 32, layout="blocked")
    with pytest.raises(ValueError):
        P.PackedTensor(u8(4, 16), u8(4, 1), None, 4, 32, scale_kind="std")
    with pytest.raises(ValueError):
        P.PackedTensor(u8(4, 15), u8(4, 1), None, 4, 30)
    with pytest.raises(ValueError):
        P.PackedTensor(u8(4, 16), u8(4, 2), None, 4, 32)
    with pytest.raises(ValueError):
        P.PackedTensor(u8(4, 16).float(), u8(4, 1), None, 4, 32)
    with pytest.raises(ValueError):
        P.PackedTensor(u8(4, 16), u8(4, 1), None, 4, 32, layout="tiled")


def test_dequantize_needs_the_gpu():
    from quartet_amd._lib import QuartetHipError
    p = P.PackedTensor(torch.zeros(4, 16, dtype=torch.uint8), torch.zeros(4, 1, dtype=torch.uint8), None, 4, 32)
    with pytest.raises(QuartetHipError):
        p.dequantize()
