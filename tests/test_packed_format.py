"""The on-disk container of a W2 weight: what is written is read back bit for bit, damage is noticed."""
import numpy as np
import pytest

from slimkernels_amd import load_w2, prepare_w2, save_w2
from slimkernels_amd.packed_format import MAGIC, read_header


def _weight(N, K, g, mode, seed=0):
    rng = np.random.default_rng(seed)
    w = rng.normal(0, 0.02, (N, K)).astype(np.float16)
    return prepare_w2(w, g, mode)


@pytest.mark.parametrize("N,K,g,mode", [(64, 256, 128, "sym"), (12, 128, 64, "ref"), (100, 512, 128, "asym"),
                                        (7, 256, 256, "asym")])
@pytest.mark.parametrize("mmap", [False, True])
def test_round_trip(tmp_path, N, K, g, mode, mmap):
    packed, scales, zero = _weight(N, K, g, mode)
    path = tmp_path / "w.w2pk"
    save_w2(path, packed, scales, zero if mode == "asym" else None, g, mode)
    f = load_w2(path, mmap=mmap)
    np.testing.assert_array_equal(np.asarray(f["packed"]), packed)
    np.testing.assert_array_equal(np.asarray(f["scales"]).view(np.uint16), scales.view(np.uint16))
    assert (f["N"], f["K"], f["group_size"], f["mode"]) == (N, K, g, mode)
    if mode == "asym":
        np.testing.assert_array_equal(f["zp"], zero)
        assert f["zp_const"] is None
        # four zero-points per byte when N allows it, one per byte otherwise
        assert read_header(path)["zp"] == ("packed2" if N % 4 == 0 else "uint8")
    else:
        assert f["zp"] is None
        assert f["zp_const"] == {"sym": 2, "ref": 1}[mode]
    for name, (offset, _) in read_header(path)["sections"].items():
        assert offset % 64 == 0, name


def test_rejects_bad_arguments(tmp_path):
    packed, scales, zero = _weight(16, 256, 128, "asym")
    with pytest.raises(ValueError):
        save_w2(tmp_path / "a", packed.astype(np.int8), scales)
    with pytest.raises(ValueError):
        save_w2(tmp_path / "a", packed, scales.astype(np.float32))
    with pytest.raises(ValueError):
        save_w2(tmp_path / "a", packed, scales, group_size=64)          # scales do not match the groups
    with pytest.raises(ValueError):
        save_w2(tmp_path / "a", packed, scales, zero + 4)              # zero-points out of range
    with pytest.raises(ValueError):
        save_w2(tmp_path / "a", packed, scales, None, 128, "custom")   # no zero-point given at all
    save_w2(tmp_path / "a", packed, scales, None, 128, "custom", zp_const=3)
    assert load_w2(tmp_path / "a")["zp_const"] == 3


def test_notices_damage(tmp_path):
    packed, scales, zero = _weight(32, 512, 128, "asym")
    path = tmp_path / "w.w2pk"
    save_w2(path, packed, scales, zero, 128, "asym")
    raw = bytearray(path.read_bytes())
    bad_magic = tmp_path / "m"
    bad_magic.write_bytes(b"X" + bytes(raw[1:]))
    with pytest.raises(ValueError, match="magic"):
        load_w2(bad_magic)
    offset = read_header(path)["sections"]["packed"][0]
    flipped = bytearray(raw)
    flipped[offset + 5] ^= 0x10
    bad_payload = tmp_path / "p"
    bad_payload.write_bytes(bytes(flipped))
    with pytest.raises(ValueError, match="checksum"):
        load_w2(bad_payload)
    assert load_w2(bad_payload, verify=False)["packed"][0, 5] != packed[0, 5]
    short = tmp_path / "s"
    short.write_bytes(bytes(raw[: offset + 10]))
    with pytest.raises(ValueError):
        load_w2(short)
    assert raw[:8] == MAGIC


@pytest.mark.gpu
def test_layer_from_file_matches_layer_from_arrays(tmp_path):
    import torch
    from slimkernels_amd import torch as ops
    for mode in ("sym", "asym"):
        packed, scales, zero = _weight(192, 1024, 128, mode, seed=3)
        path = tmp_path / f"{mode}.w2pk"
        save_w2(path, packed, scales, zero if mode == "asym" else None, 128, mode)
        direct = ops.repack_w2(packed, scales, zero if mode == "asym" else None, 128, zp_const=2 if mode == "sym" else 0)
        loaded = ops.load_w2_weight(path)
        assert torch.equal(direct.w_r, loaded.w_r) and torch.equal(direct.s_r, loaded.s_r)
        assert (direct.zp_r is None) == (loaded.zp_r is None) and direct.zp_const == loaded.zp_const
        if direct.zp_r is not None:
            assert torch.equal(direct.zp_r, loaded.zp_r)
        x = torch.randn(5, 1024, device="cuda", dtype=torch.float16)
        y0 = ops.W2A8Linear(direct)(x)
        y1 = ops.W2A8Linear.from_file(path)(x)
        assert torch.equal(y0, y1)
