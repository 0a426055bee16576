"""Minimal reader for the ONNX TensorProto files (`input_i.pb`, `output_i.pb`) kept under
tests/golden/single_op/: the data files of the reference's own single-op tests
(tests/single_op.rs there).  Only the fields those files use are decoded:
  1 dims (varint, packed or not), 2 data_type, 8 name, 9 raw_data,
  4 float_data / 5 int32_data / 7 int64_data (packed) as a fallback.
bf16 tensors come back as uint16 bit patterns plus their f32 widening.
"""
import struct

import numpy as np

ONNX_F32, ONNX_U8, ONNX_I8, ONNX_I32, ONNX_I64, ONNX_BF16, ONNX_F16, ONNX_F64 = 1, 2, 3, 6, 7, 16, 10, 11


def _varint(buf, pos):
    result = 0
    shift = 0
    while True:
        b = buf[pos]
        pos += 1
        result |= (b & 0x7F) << shift
        if not b & 0x80:
            return result, pos
        shift += 7


def _signed64(u):
    return u - (1 << 64) if u >= (1 << 63) else u


class PbTensor:
    def __init__(self, dims, data_type, name, array):
        self.dims = dims
        self.data_type = data_type
        self.name = name
        self.array = array  # numpy array in the storage type (bf16/f16 -> uint16 bits)

    def f32(self):
        """Values widened to float32 (exact for bf16/f16/int8)."""
        if self.data_type == ONNX_BF16:
            return (self.array.astype(np.uint32) << 16).view(np.float32)
        if self.data_type == ONNX_F16:
            return self.array.view(np.float16).astype(np.float32)
        return self.array.astype(np.float32)


def read_tensor(path):
    with open(path, "rb") as f:
        buf = f.read()
    pos = 0
    dims = []
    data_type = None
    name = ""
    raw = None
    floats, i32s, i64s = [], [], []
    while pos < len(buf):
        key, pos = _varint(buf, pos)
        field, wire = key >> 3, key & 7
        if wire == 0:
            val, pos = _varint(buf, pos)
            if field == 1:
                dims.append(_signed64(val))
            elif field == 2:
                data_type = val
            elif field == 5:
                i32s.append(_signed64(val))
            elif field == 7:
                i64s.append(_signed64(val))
        elif wire == 2:
            ln, pos = _varint(buf, pos)
            chunk = buf[pos:pos + ln]
            pos += ln
            if field == 1:
                p = 0
                while p < len(chunk):
                    v, p = _varint(chunk, p)
                    dims.append(_signed64(v))
            elif field == 8:
                name = chunk.decode("utf-8")
            elif field == 9:
                raw = chunk
            elif field == 4:
                floats.extend(struct.unpack("<%df" % (len(chunk) // 4), chunk))
            elif field in (5, 7):
                p = 0
                dst = i32s if field == 5 else i64s
                while p < len(chunk):
                    v, p = _varint(chunk, p)
                    dst.append(_signed64(v))
        elif wire == 5:
            if field == 4:
                floats.append(struct.unpack("<f", buf[pos:pos + 4])[0])
            pos += 4
        elif wire == 1:
            pos += 8
        else:
            raise ValueError("unsupported wire type %d in %s" % (wire, path))
    np_types = {ONNX_F32: np.float32, ONNX_U8: np.uint8, ONNX_I8: np.int8, ONNX_I32: np.int32,
                ONNX_I64: np.int64, ONNX_BF16: np.uint16, ONNX_F16: np.uint16, ONNX_F64: np.float64}
    if data_type not in np_types:
        raise ValueError("unsupported ONNX data_type %r in %s" % (data_type, path))
    dt = np_types[data_type]
    if raw is not None:
        arr = np.frombuffer(raw, dtype=dt).copy()
    elif floats:
        arr = np.asarray(floats, dtype=dt)
    elif i64s:
        arr = np.asarray(i64s, dtype=dt)
    elif i32s:
        # int32_data also carries (u)int8/16 and bf16/f16 bit patterns
        arr = np.asarray(i32s, dtype=np.int64).astype(dt)
    else:
        arr = np.zeros(0, dtype=dt)
    arr = arr.reshape(dims) if dims else arr.reshape(())
    return PbTensor(dims, data_type, name, arr)


def read_case(case_dir):
    """Returns (inputs, outputs): lists of PbTensor ordered by file index."""
    import glob
    import os
    import re

    def idx(p):
        return int(re.search(r"_(\d+)\.pb$", p).group(1))

    ins = sorted(glob.glob(os.path.join(case_dir, "input_*.pb")), key=idx)
    outs = sorted(glob.glob(os.path.join(case_dir, "output_*.pb")), key=idx)
    return [read_tensor(p) for p in ins], [read_tensor(p) for p in outs]
