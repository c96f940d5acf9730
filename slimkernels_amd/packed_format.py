"""On-disk container for a W2 weight in the interchange layout.

What is stored is exactly what the host-side preparation produces and what
``slimkernels_amd.torch.repack_w2`` consumes: the packed 2-bit codes ``[N, K/4]`` uint8 in the
pack_matrix byte order (upstream matrix_packer.py:33-34: four codes per byte along K, first code
in the two high bits), the group scales ``[G, N]`` float16 in the quantize layout (upstream
quantization.py:53: groups along K, one row per group), and, for per-group zero-points, their
``[G, N]`` values packed four per byte along N with the same rule.  The gfx950 streaming layout is
never written to disk: it is private to one library version and is rebuilt at load time.

File layout (little endian):
    bytes 0..7    magic  b"SLIMW2PK"
    bytes 8..11   uint32 length of the header text
    header        UTF-8 JSON: version, N, K, group_size, mode, zp_const, zp ("none" | "packed2" |
                  "uint8"), sections {name: [offset, nbytes]}, crc32 of the payload
    payload       the sections, each starting on a 64-byte boundary of the file
"""
import json
import struct
import zlib

import numpy as np

from .matrix_packer import pack_matrix, unpack_matrix

MAGIC = b"SLIMW2PK"
VERSION = 1
_ALIGN = 64


def _align(n):
    return (n + _ALIGN - 1) // _ALIGN * _ALIGN


def save_w2(path, packed, scales, zp=None, group_size=128, mode="sym", zp_const=None):
    """Write one weight.  ``packed`` uint8 [N, K/4], ``scales`` float16 [G, N], ``zp`` uint8 [G, N] with
    values 0..3 or None; without ``zp`` every zero-point is ``zp_const`` (default: 2 for mode "sym",
    1 for "ref").  ``mode`` is a tag for the reader ("sym", "ref", "asym" or any other string)."""
    packed = np.ascontiguousarray(packed)
    scales = np.ascontiguousarray(scales)
    if packed.dtype != np.uint8 or packed.ndim != 2:
        raise ValueError("packed must be a 2-D uint8 array [N, K/4]")
    if scales.dtype != np.float16 or scales.ndim != 2:
        raise ValueError("scales must be a 2-D float16 array [G, N]")
    N, K = packed.shape[0], packed.shape[1] * 4
    if group_size <= 0 or K % group_size != 0 or scales.shape != (K // group_size, N):
        raise ValueError(f"scales shape {scales.shape} does not match (K/group_size, N) = ({K // max(group_size, 1)}, {N})")
    sections = [("packed", packed.tobytes()), ("scales", scales.tobytes())]
    zp_kind = "none"
    if zp is not None:
        zp = np.ascontiguousarray(zp)
        if zp.dtype != np.uint8 or zp.shape != scales.shape:
            raise ValueError("zp must be uint8 with the shape of scales")
        if zp.size and int(zp.max()) > 3:
            raise ValueError("zero-points must be in 0..3")
        if N % 4 == 0:
            zp_kind = "packed2"
            sections.append(("zp", pack_matrix(zp).tobytes()))
        else:
            zp_kind = "uint8"
            sections.append(("zp", zp.tobytes()))
    elif zp_const is None:
        zp_const = {"sym": 2, "ref": 1}.get(mode)
        if zp_const is None:
            raise ValueError("without zp, zp_const must be given for this mode")
    if zp_const is not None and not 0 <= int(zp_const) <= 3:
        raise ValueError("zp_const must be in 0..3")

    crc = 0
    for _, blob in sections:
        crc = zlib.crc32(blob, crc)
    header = {"version": VERSION, "N": N, "K": K, "group_size": int(group_size), "mode": str(mode),
              "zp_const": None if zp is not None else int(zp_const), "zp": zp_kind, "crc32": crc, "sections": {}}
    # the header's own length decides the offsets, and the offsets are in the header: place the sections
    # for a header padded to a fixed size (a few hundred bytes are plenty)
    reserve = 1024
    while True:
        offset = _align(len(MAGIC) + 4 + reserve)
        for name, blob in sections:
            header["sections"][name] = [offset, len(blob)]
            offset = _align(offset + len(blob))
        text = json.dumps(header, sort_keys=True).encode("utf-8")
        if len(text) <= reserve:
            break
        reserve *= 2
    text = text + b" " * (reserve - len(text))
    with open(path, "wb") as f:
        f.write(MAGIC)
        f.write(struct.pack("<I", len(text)))
        f.write(text)
        for name, blob in sections:
            f.seek(header["sections"][name][0])
            f.write(blob)
        f.truncate(_align(f.tell()))


def read_header(path):
    """The header of a file written by save_w2 (a dict), after checking magic and version."""
    with open(path, "rb") as f:
        head = f.read(len(MAGIC) + 4)
        if len(head) < len(MAGIC) + 4 or head[:len(MAGIC)] != MAGIC:
            raise ValueError(f"{path}: not a packed W2 weight file (bad magic)")
        (n,) = struct.unpack("<I", head[len(MAGIC):])
        text = f.read(n)
    if len(text) != n:
        raise ValueError(f"{path}: truncated header")
    try:
        header = json.loads(text.decode("utf-8"))
    except (UnicodeDecodeError, json.JSONDecodeError) as e:
        raise ValueError(f"{path}: unreadable header ({e})") from None
    if header.get("version") != VERSION:
        raise ValueError(f"{path}: file version {header.get('version')!r}, this reader knows {VERSION}")
    return header


def load_w2(path, mmap=False, verify=True):
    """Read one weight.  Returns a dict with ``packed`` uint8 [N, K/4], ``scales`` float16 [G, N], ``zp``
    uint8 [G, N] or None, and ``group_size``, ``mode``, ``zp_const`` (None when ``zp`` is present), ``N``,
    ``K``.  ``mmap=True`` maps the two large arrays instead of reading them; ``verify`` checks the CRC."""
    header = read_header(path)
    N, K, g = header["N"], header["K"], header["group_size"]
    G = K // g
    want = {"packed": N * (K // 4), "scales": 2 * G * N}
    if header["zp"] == "packed2":
        want["zp"] = G * (N // 4)
    elif header["zp"] == "uint8":
        want["zp"] = G * N
    elif header["zp"] != "none":
        raise ValueError(f"{path}: unknown zero-point storage {header['zp']!r}")
    for name, nbytes in want.items():
        sec = header["sections"].get(name)
        if sec is None or sec[1] != nbytes:
            raise ValueError(f"{path}: section {name!r} is missing or has the wrong size")

    def section(name, dtype, shape):
        offset, nbytes = header["sections"][name]
        if mmap:
            return np.memmap(path, dtype=dtype, mode="r", offset=offset, shape=shape)
        with open(path, "rb") as f:
            f.seek(offset)
            blob = f.read(nbytes)
        if len(blob) != nbytes:
            raise ValueError(f"{path}: truncated section {name!r}")
        return np.frombuffer(blob, dtype=dtype).reshape(shape)

    packed = section("packed", np.uint8, (N, K // 4))
    scales = section("scales", np.float16, (G, N))
    zp_raw = None
    if header["zp"] == "packed2":
        zp_raw = section("zp", np.uint8, (G, N // 4))
    elif header["zp"] == "uint8":
        zp_raw = section("zp", np.uint8, (G, N))
    if verify:
        crc = zlib.crc32(packed)
        crc = zlib.crc32(scales, crc)
        if zp_raw is not None:
            crc = zlib.crc32(zp_raw, crc)
        if crc != header["crc32"]:
            raise ValueError(f"{path}: payload checksum mismatch (file damaged)")
    zp = None
    if header["zp"] == "packed2":
        zp = unpack_matrix(np.ascontiguousarray(zp_raw))
    elif header["zp"] == "uint8":
        zp = zp_raw
    return {"packed": packed, "scales": scales, "zp": zp, "group_size": g, "mode": header["mode"],
            "zp_const": header["zp_const"], "N": N, "K": K}
