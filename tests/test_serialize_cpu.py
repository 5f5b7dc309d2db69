"""The .nnue codec: signed LEB128 against the published examples of the encoding, the file against its
own reader (a fixed point of write -> read -> write), and the tensors in the file against the
quantization functions of the int16 / int8 path."""
import io
import struct

import numpy as np
import pytest
import torch

from nnueft import model as M
from nnueft import quantized
from nnueft import serialize as S

CFG = dict(L1=64, L2=15, L3=32)


def _model(seed=0):
    torch.manual_seed(seed)
    m = M.NNUEModel("HalfKAv2_hm^", M.ModelConfig(**CFG))
    with torch.no_grad():
        m.input.features[0].virtual_weight.normal_(0, 0.01)
        m.layer_stacks.l1.factorized_linear.weight.normal_(0, 0.01)
        m.layer_stacks.l1.factorized_linear.bias.normal_(0, 0.01)
    return m


def test_leb128_known_encodings():
    # signed LEB128 as defined by the DWARF standard (its worked examples) and the values around the
    # one-byte boundary
    known = [(2, b"\x02"), (-2, b"\x7e"), (127, b"\xff\x00"), (-127, b"\x81\x7f"), (128, b"\x80\x01"),
             (-128, b"\x80\x7f"), (129, b"\x81\x01"), (-129, b"\xff\x7e"), (0, b"\x00"), (-1, b"\x7f"),
             (63, b"\x3f"), (64, b"\xc0\x00"), (-64, b"\x40"), (-65, b"\xbf\x7f"), (-123456, b"\xc0\xbb\x78")]
    for v, enc in known:
        assert S.encode_leb_128_array(np.array([v])) == enc, v
        assert S.decode_leb_128_array(enc, 1).tolist() == [v]
    assert S.encode_leb_128_array(np.array([v for v, _ in known])) == b"".join(e for _, e in known)


def test_leb128_round_trip_and_truncation():
    rng = np.random.default_rng(0)
    a = np.concatenate([rng.integers(-2 ** 31, 2 ** 31, size=5000), rng.integers(-300, 300, size=5000),
                        [0, -1, 2 ** 31 - 1, -2 ** 31, 32767, -32768]])
    enc = S.encode_leb_128_array(a)
    assert np.array_equal(S.decode_leb_128_array(enc, len(a)), a)
    assert np.array_equal(S.decode_leb_128_array(enc, 10), a[:10])
    with pytest.raises(EOFError):
        S.decode_leb_128_array(enc[:-1], len(a))
    assert S.encode_leb_128_array(np.zeros(0, np.int16)) == b"" and len(S.decode_leb_128_array(b"", 0)) == 0


@pytest.mark.parametrize("compression", ["none", "leb128"])
def test_file_is_a_fixed_point_and_holds_the_quantized_tensors(compression):
    m = _model()
    w = S.NNUEWriter(m, "a test net", compression)
    buf = bytes(w.buf)
    # header fields by position
    version, net_hash, dlen = struct.unpack_from("<III", buf, 0)
    assert version == 0x6A448AFA and buf[12:12 + dlen] == b"a test net"
    (ft_hash,) = struct.unpack_from("<I", buf, 12 + dlen)
    assert ft_hash == (m.input.HASH ^ 128) and net_hash == (S.NNUEWriter.fc_hash(m) ^ m.input.HASH ^ 128)
    r = S.NNUEReader(io.BytesIO(buf), "HalfKAv2_hm^", M.ModelConfig(**CFG))
    assert r.description == "a test net"
    assert bytes(S.NNUEWriter(r.model, "a test net", compression).buf) == buf
    # what the file holds is what the quantized path evaluates
    export = m.input.get_export_weights()
    w16, b16, p32 = quantized.quantize_feature_transformer(export, m.input.bias.data, 64)
    e2 = r.model.input.get_export_weights()
    w16r, b16r, p32r = quantized.quantize_feature_transformer(e2, r.model.input.bias.data, 64)
    assert torch.equal(w16, w16r) and torch.equal(b16, b16r) and torch.equal(p32, p32r)
    for a, b in zip(quantized.quantize_layer_stacks(m.layer_stacks), quantized.quantize_layer_stacks(r.model.layer_stacks)):
        assert torch.equal(a, b)
    if compression == "none":
        # raw layout: bias right behind the feature transformer hash, then the 22528 x 64 int16 table
        at = 16 + dlen
        assert np.array_equal(np.frombuffer(buf, "<i2", 64, at), b16.numpy())
        assert np.array_equal(np.frombuffer(buf, "<i2", 22528 * 64, at + 128).reshape(22528, 64), w16.numpy())
        at += 128 + 22528 * 64 * 2
        assert np.array_equal(np.frombuffer(buf, "<i4", 22528 * 8, at).reshape(22528, 8), p32.numpy())
        at += 22528 * 8 * 4
        # first bucket: hash, l1 bias int32[15], l1 weight int8[15, 64], l2 bias [32], l2 weight [32, 32 (30 padded)]
        assert struct.unpack_from("<I", buf, at)[0] == S.NNUEWriter.fc_hash(m)
        w1, b1, w2, b2, wo, bo = quantized.quantize_layer_stacks(m.layer_stacks)
        assert np.array_equal(np.frombuffer(buf, "<i4", 15, at + 4), b1[:15].numpy())
        assert np.array_equal(np.frombuffer(buf, "i1", 15 * 64, at + 64).reshape(15, 64), w1[:15].numpy())
        at += 64 + 15 * 64
        assert np.array_equal(np.frombuffer(buf, "<i4", 32, at), b2[:32].numpy())
        l2w = np.frombuffer(buf, "i1", 32 * 32, at + 128).reshape(32, 32)
        assert np.array_equal(l2w[:, :30], w2[:32].numpy()) and not l2w[:, 30:].any()
        # total size: header, FT, 8 buckets of (hash + three layers with inputs padded to 32)
        per_bucket = 4 + (15 * 4 + 15 * 64) + (32 * 4 + 32 * 32) + (4 + 96)
        assert len(buf) == 16 + dlen + 128 + 22528 * 64 * 2 + 22528 * 8 * 4 + 8 * per_bucket


def test_reader_rejects_another_architecture_and_a_short_file():
    m = _model()
    buf = bytes(S.NNUEWriter(m, "x").buf)
    with pytest.raises(ValueError, match="Expected"):
        S.NNUEReader(io.BytesIO(buf), "HalfKAv2_hm^", M.ModelConfig(L1=128, L2=15, L3=32))
    with pytest.raises(EOFError):
        S.NNUEReader(io.BytesIO(buf[:-5]), "HalfKAv2_hm^", M.ModelConfig(**CFG))
    with pytest.raises(ValueError):
        S.NNUEWriter(m, "x", "zip")
