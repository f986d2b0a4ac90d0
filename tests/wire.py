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


# ---- reader for the same subset (tests only): NetParameter -> {layer name: [arrays]} ------------

def _fields(buf):
    """Yields (field number, wire type, value) of one message; value is an int or bytes."""
    i = 0
    while i < len(buf):
        k = 0
        shift = 0
        while True:
            b = buf[i]
            i += 1
            k |= (b & 0x7F) << shift
            shift += 7
            if b < 0x80:
                break
        number, wt = k >> 3, k & 7
        if wt == 0:
            v = 0
            shift = 0
            while True:
                b = buf[i]
                i += 1
                v |= (b & 0x7F) << shift
                shift += 7
                if b < 0x80:
                    break
            yield number, wt, v
        elif wt == 2:
            n = 0
            shift = 0
            while True:
                b = buf[i]
                i += 1
                n |= (b & 0x7F) << shift
                shift += 7
                if b < 0x80:
                    break
            yield number, wt, bytes(buf[i:i + n])
            i += n
        elif wt == 5:
            yield number, wt, bytes(buf[i:i + 4])
            i += 4
        elif wt == 1:
            yield number, wt, bytes(buf[i:i + 8])
            i += 8
        else:
            raise ValueError("wire type %d" % wt)


def _varints(buf):
    out, v, shift = [], 0, 0
    for b in buf:
        v |= (b & 0x7F) << shift
        shift += 7
        if b < 0x80:
            out.append(v)
            v, shift = 0, 0
    return out


def read_net_blobs(buf):
    """Layer parameter blobs of a binary NetParameter written with `layer` (field 100):
    {layer name: [float32 arrays shaped by BlobProto.shape (7) or num..width (1-4)]}."""
    import numpy as np
    out = {}
    for number, wt, v in _fields(buf):
        if number != 100 or wt != 2:
            continue
        name, blobs = None, []
        for n2, w2, v2 in _fields(v):
            if n2 == 1 and w2 == 2:
                name = v2.decode()
            elif n2 == 7 and w2 == 2:
                data, shape, legacy = [], None, {}
                for n3, w3, v3 in _fields(v2):
                    if n3 == 5 and w3 == 2:
                        data.append(np.frombuffer(v3, "<f4"))
                    elif n3 == 5 and w3 == 5:
                        data.append(np.frombuffer(v3, "<f4"))
                    elif n3 == 7 and w3 == 2:
                        dims = []
                        for n4, w4, v4 in _fields(v3):
                            if n4 == 1 and w4 == 0:
                                dims.append(v4)
                            elif n4 == 1 and w4 == 2:   # packed dims
                                dims.extend(_varints(v4))
                        shape = dims
                    elif n3 in (1, 2, 3, 4) and w3 == 0:
                        legacy[n3] = v3
                arr = np.concatenate(data) if data else np.zeros(0, np.float32)
                if shape is None and legacy:
                    shape = [legacy.get(k, 1) for k in (1, 2, 3, 4)]
                blobs.append(arr.reshape(shape) if shape else arr)
        if blobs:
            out[name] = blobs
    return out
