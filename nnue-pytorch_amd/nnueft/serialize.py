"""Reader and writer of the .nnue file the engine loads: the wire format of the quantized tensors
the int16 / int8 kernels of this build evaluate.

Layout (all little endian), following NNUEWriter / NNUEReader of the reference
(model/utils/serialize.py:102-400):

    u32 version (0x6A448AFA)        u32 network hash = fc_hash ^ feature_hash ^ (2 * L1)
    u32 length of the description, then its UTF-8 bytes
    u32 feature transformer hash = feature_hash ^ (2 * L1)
    int16 bias[L1]                                       (tensor, see below)
    per feature block: int16 weight[rows, L1], int32 psqt[rows, n_psqt]     rows = 22528, kings merged
    per layer-stack bucket: u32 fc_hash, then for each of the three layers int32 bias[out] and
    int8 weight[out, in padded to a multiple of 32]       (never compressed)
    a tensor is either its raw bytes or the 17 bytes "COMPRESSED_LEB128", a u32 byte count and the
    values as signed LEB128.

No numba here: the LEB128 codec is vectorised numpy (at most five bytes per 32-bit value).
"""
import struct
from functools import reduce
import operator

import numpy as np
import torch

from . import model as M

VERSION = 0x6A448AFA
DEFAULT_DESCRIPTION = "Network trained with the https://github.com/official-stockfish/nnue-pytorch trainer."
LEB128_MAGIC = b"COMPRESSED_LEB128"


def encode_leb_128_array(arr) -> bytes:
    """Signed LEB128 of every value of an integer array, concatenated (serialize.py:64-75)."""
    v = np.asarray(arr).astype(np.int64).ravel()
    n = v.size
    out = np.zeros((n, 10), np.uint8)
    length = np.zeros(n, np.int64)
    alive = np.ones(n, bool)
    for k in range(10):
        byte = (v & 0x7F).astype(np.uint8)
        v = v >> 7                                    # arithmetic shift: -1 stays -1
        sign = (byte & 0x40) != 0
        last = ((v == 0) & ~sign) | ((v == -1) & sign)
        out[:, k] = np.where(alive, np.where(last, byte, byte | 0x80), 0)
        length = np.where(alive, k + 1, length)
        alive &= ~last
        if not alive.any():
            break
    keep = np.arange(10)[None, :] < length[:, None]
    return out[keep].tobytes()


def decode_leb_128_array(data: bytes, n: int) -> np.ndarray:
    """The first n signed LEB128 values of `data` as int64 (serialize.py:78-94)."""
    b = np.frombuffer(data, np.uint8)
    ends = np.nonzero((b & 0x80) == 0)[0]
    if len(ends) < n:
        raise EOFError("Unexpected end of LEB128 data.")
    ends = ends[:n]
    starts = np.concatenate([[0], ends[:-1] + 1]) if n else np.zeros(0, np.int64)
    length = ends - starts + 1
    if n and int(length.max()) > 10:
        raise ValueError("LEB128 value longer than 64 bits.")
    value = np.zeros(n, np.int64)
    for k in range(int(length.max()) if n else 0):
        has = length > k
        byte = np.where(has, b[np.minimum(starts + k, len(b) - 1)], 0).astype(np.int64)
        value |= (byte & 0x7F) << (7 * k)
    shift = 7 * length
    negative = (b[ends] & 0x40) != 0
    fill = np.where(shift < 64, -(np.int64(1) << np.minimum(shift, 62)), 0)
    return np.where(negative, value | fill, value)


def _quantize(value: torch.Tensor, scale: float, dtype: torch.dtype) -> torch.Tensor:
    from .quantized import _safe_round_to

    return _safe_round_to(value.detach().float().cpu() * scale, dtype)


class NNUEWriter:
    """buf = the .nnue image of `model` (nnueft.model.NNUEModel)."""

    def __init__(self, model, description=None, ft_compression: str = "none"):
        if ft_compression not in ("none", "leb128"):
            raise ValueError("Invalid compression method.")
        self.buf = bytearray()
        fc_hash = self.fc_hash(model)
        feature_hash = model.input.HASH
        desc = (DEFAULT_DESCRIPTION if description is None else description).encode("utf-8")
        self.int32(VERSION)
        self.int32(fc_hash ^ feature_hash ^ (model.L1 * 2))
        self.int32(len(desc))
        self.buf.extend(desc)
        self.int32(feature_hash ^ (model.L1 * 2))
        self.write_feature_transformer(model, ft_compression)
        ls = model.layer_stacks
        for bucket in range(ls.count):
            self.int32(fc_hash)
            for layer in (ls.l1, ls.l2, ls.output):
                self.write_fc_layer(model, layer.at_index(bucket), layer.layer_key)

    @staticmethod
    def fc_hash(model) -> int:
        """Hash of the layer-stack architecture (serialize.py:132-154)."""
        prev = 0xEC42E90D ^ (model.L1 * 2)
        layer_hash = prev
        for layer in (model.layer_stacks.l1, model.layer_stacks.l2, model.layer_stacks.output):
            outs = layer.out_features
            layer_hash = 0xCC03DAE4 + outs
            layer_hash ^= prev >> 1
            layer_hash ^= (prev << 31) & 0xFFFFFFFF
            if outs != 1:
                layer_hash = (layer_hash + 0x538D24C7) & 0xFFFFFFFF     # clipped ReLU behind it
            prev = layer_hash
        return layer_hash

    def int32(self, v: int) -> None:
        self.buf.extend(struct.pack("<I", v & 0xFFFFFFFF))

    def write_tensor(self, t: torch.Tensor, compression: str = "none") -> None:
        arr = t.detach().flatten().cpu().numpy()
        if compression == "none":
            self.buf.extend(arr.astype(arr.dtype.newbyteorder("<")).tobytes())
        else:
            self.buf.extend(LEB128_MAGIC)
            body = encode_leb_128_array(arr)
            self.int32(len(body))
            self.buf.extend(body)

    def write_feature_transformer(self, model, ft_compression: str) -> None:
        q = model.quantization.weight_scales_dict
        ft = model.input
        self.write_tensor(_quantize(ft.bias.data[: model.L1], q["ft_bias"], torch.int16), ft_compression)
        export = ft.get_export_weights()
        at = 0
        for f in ft.features:
            seg = export[at:at + f.NUM_REAL_FEATURES]
            at += f.NUM_REAL_FEATURES
            self.write_tensor(_quantize(seg[:, : model.L1], q["ft_weight"], torch.int16), ft_compression)
            self.write_tensor(_quantize(seg[:, model.L1:], q["ft_psqt_weight"], torch.int32), ft_compression)

    def write_fc_layer(self, model, layer, layer_key: str) -> None:
        q = model.quantization.weight_scales_dict
        bias = _quantize(layer.bias.data, q[f"{layer_key}_bias"], torch.int32)
        weight = _quantize(layer.weight.data, q[f"{layer_key}_weight"], torch.int8)
        pad = (-weight.shape[1]) % 32          # inputs padded to a multiple of 32
        if pad:
            weight = torch.cat([weight, torch.zeros(weight.shape[0], pad, dtype=torch.int8)], dim=1)
        self.write_tensor(bias)
        self.write_tensor(weight)


class NNUEReader:
    """model = the float NNUEModel whose export is the file (virtual weights zero), description = its text."""

    def __init__(self, f, feature_name: str, config):
        self.f = f
        self.model = M.NNUEModel(feature_name, config)
        self.config = config
        m = self.model
        fc_hash = NNUEWriter.fc_hash(m)
        feature_hash = m.input.HASH
        self.read_int32(VERSION)
        self.read_int32(fc_hash ^ feature_hash ^ (config.L1 * 2))
        self.description = self.f.read(self.read_int32()).decode("utf-8")
        self.read_int32(feature_hash ^ (config.L1 * 2))
        m.zero_virtual_weights()
        self.read_feature_transformer()
        ls = m.layer_stacks
        for bucket in range(ls.count):
            self.read_int32(fc_hash)
            for layer in (ls.l1, ls.l2, ls.output):
                self.read_fc_layer(layer, bucket)

    def read_int32(self, expected=None) -> int:
        raw = self.f.read(4)
        if len(raw) != 4:
            raise EOFError("Unexpected end of file.")
        v = struct.unpack("<I", raw)[0]
        if expected is not None and v != (expected & 0xFFFFFFFF):
            raise ValueError(f"Expected: {expected & 0xFFFFFFFF:x}, got: {v:x}")
        return v

    def tensor(self, dtype, shape) -> torch.Tensor:
        count = reduce(operator.mul, shape, 1)
        pos = self.f.tell()
        if self.f.read(len(LEB128_MAGIC)) == LEB128_MAGIC:
            nbytes = self.read_int32()
            body = self.f.read(nbytes)
            if len(body) != nbytes:
                raise EOFError("Unexpected end of file when reading compressed data.")
            values = decode_leb_128_array(body, count)
        else:
            self.f.seek(pos)
            dt = np.dtype(dtype).newbyteorder("<")
            raw = self.f.read(count * dt.itemsize)
            if len(raw) != count * dt.itemsize:
                raise EOFError("Unexpected end of file.")
            values = np.frombuffer(raw, dt)
        return torch.from_numpy(values.astype(np.float32)).reshape(list(shape))

    def read_feature_transformer(self) -> None:
        m, ft = self.model, self.model.input
        q = m.quantization.weight_scales_dict
        L1, n_psqt = m.L1, m.num_psqt_buckets
        bias = self.tensor(np.int16, [L1]) / q["ft_bias"]
        rows = []
        for f in ft.features:
            w = self.tensor(np.int16, [f.NUM_REAL_FEATURES, L1]) / q["ft_weight"]
            p = self.tensor(np.int32, [f.NUM_REAL_FEATURES, n_psqt]) / q["ft_psqt_weight"]
            rows.append(torch.cat([w, p], dim=1))
        ft.bias.data = torch.cat([bias, torch.zeros(n_psqt)])
        ft.load_export_weights(torch.cat(rows, dim=0))

    def read_fc_layer(self, layer, bucket: int) -> None:
        q = self.model.quantization.weight_scales_dict
        outs, ins = layer.out_features, layer.in_features
        bias = self.tensor(np.int32, [outs]) / q[f"{layer.layer_key}_bias"]
        weight = self.tensor(np.int8, [outs, (ins + 31) // 32 * 32]) / q[f"{layer.layer_key}_weight"]
        lo, hi = bucket * outs, (bucket + 1) * outs
        with torch.no_grad():
            layer.linear.bias[lo:hi] = bias
            layer.linear.weight[lo:hi] = weight[:, :ins]
