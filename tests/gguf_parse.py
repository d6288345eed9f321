"""A reader of GGUF v3 files written from the published layout, independent of the writer under test:
header, typed key/value pairs, tensor directory, aligned data section."""
import struct

import numpy as np

_SCALARS = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}
_GGML_NUMPY = {0: np.float32, 1: np.float16, 24: np.int8, 25: np.int16, 26: np.int32, 27: np.int64, 28: np.float64}


def parse_gguf(path):
    """-> (version, [(key, value_type, value)], {name: (array, offset)}, alignment, data_start)"""
    buf = open(path, "rb").read()
    pos = 0

    def take(fmt):
        nonlocal pos
        vals = struct.unpack_from(fmt, buf, pos)
        pos += struct.calcsize(fmt)
        return vals[0] if len(vals) == 1 else vals

    def string():
        nonlocal pos
        n = take("<Q")
        s = buf[pos:pos + n]
        pos += n
        return s

    def value(vt):
        if vt in _SCALARS:
            return take(_SCALARS[vt])
        if vt == 8:
            return string()
        if vt == 9:
            et, n = take("<I"), take("<Q")
            return (et, [value(et) for _ in range(n)])
        raise AssertionError(f"value type {vt}")

    assert buf[:4] == b"GGUF"
    pos = 4
    version, n_tensors, n_kv = take("<I"), take("<Q"), take("<Q")
    kvs = []
    for _ in range(n_kv):
        key = string().decode()
        vt = take("<I")
        kvs.append((key, vt, value(vt)))
    directory = []
    for _ in range(n_tensors):
        name = string().decode()
        rank = take("<I")
        dims = [take("<Q") for _ in range(rank)]
        directory.append((name, dims, take("<I"), take("<Q")))
    alignment = dict((k, v) for k, _, v in kvs).get("general.alignment", 32)
    data_start = pos + (-pos) % alignment
    assert set(buf[pos:data_start]) <= {0}
    tensors, end = {}, data_start
    for name, dims, gt, off in directory:
        assert off % alignment == 0 and name not in tensors
        dt = np.dtype(_GGML_NUMPY[gt]).newbyteorder("<")
        count = int(np.prod(dims))
        a = np.frombuffer(buf, dtype=dt, count=count, offset=data_start + off).reshape(dims[::-1])
        tensors[name] = (a, off)
        assert data_start + off >= end                      # in directory order, no overlap
        end = data_start + off + a.nbytes
    assert len(buf) == end + (-(end - data_start)) % alignment
    return version, kvs, tensors, alignment, data_start
