"""Minimal protobuf wire-format writer for caffemodel fixtures (test side only):
NetParameter{name=1, layer=100{name=1, type=2, blobs=7{data=5 packed, shape=7{dim=1 packed}}}}
plus the legacy 4-D blob form (num=1..width=4) and double_data=8."""
import struct

import numpy as np


def varint(v):
    out = bytearray()
    v &= (1 << 64) - 1
    while v >= 0x80:
        out.append((v & 0x7F) | 0x80)
        v >>= 7
    out.append(v)
    return bytes(out)


def key(number, wt):
    return varint((number << 3) | wt)


def ld(number, payload):
    return key(number, 2) + varint(len(payload)) + payload


def blob(arr, legacy=False, as_double=False, packed=True):
    arr = np.asarray(arr)
    out = b""
    if legacy:
        shape4 = (1,) * (4 - arr.ndim) + arr.shape
        for i, d in enumerate(shape4):
            out += key(i + 1, 0) + varint(d)
    if as_double:
        out += ld(8, arr.astype("<f8").tobytes())
    elif packed:
        out += ld(5, arr.astype("<f4").tobytes())
    else:
        for v in arr.astype("<f4").ravel():
            out += key(5, 5) + struct.pack("<f", v)
    if not legacy:
        out += ld(7, ld(1, b"".join(varint(d) for d in arr.shape)))
    return out


def layer(name, type_, blobs, **kw):
    out = ld(1, name.encode()) + ld(2, type_.encode())
    # an unknown-to-the-reader field (phase = 10, varint) that must be skipped
    out += key(10, 0) + varint(1)
    for b in blobs:
        out += ld(7, blob(b, **kw))
    return out


def v1_layer(name, type_number, blobs, **kw):
    """V1LayerParameter: name = 4, type (enum) = 5, blobs = 6, blobs_lr = 7."""
    out = ld(4, name.encode()) + key(5, 0) + varint(type_number)
    for b in blobs:
        out += ld(6, blob(b, **kw)) + key(7, 5) + struct.pack("<f", 1.0)
    return out


def net(name, layers, v1_layers=()):
    out = ld(1, name.encode())
    for l in v1_layers:
        out += ld(2, l)
    for l in layers:
        out += ld(100, l)
    return out
