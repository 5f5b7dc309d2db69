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


def test_leb128_edge_values_as_the_reference_encoder_loop_gives_them():
    """The reference's encoder (model/utils/serialize.py:64-75) takes 7 bits at a time and stops when what is left is
    0 with bit 6 clear or -1 with bit 6 set.  Worked by hand for the edges of one byte and of int16:
      63: byte 0x3f, rest 0, bit 6 clear -> 3f.            64: byte 0x40, rest 0 but bit 6 set -> c0, then 00.
     -64: byte 0x40, rest -1, bit 6 set -> 40.            -65: byte 0x3f, rest -1 but bit 6 clear -> bf, then 7f.
    32767: 7f|80, 7f|80, then 01 (rest 0, bit 6 clear).  -32768: 00|80, 00|80, then 7e (rest -1, bit 6 set)."""
    hand = [(63, "3f"), (64, "c000"), (-64, "40"), (-65, "bf7f"), (32767, "ffff01"), (-32768, "80807e"),
            (8191, "ff3f"), (8192, "80c000"), (-8192, "8040"), (-8193, "ffbf7f")]
    for v, hexbytes in hand:
        assert S.encode_leb_128_array(np.array([v], np.int16)).hex() == hexbytes, v
        assert S.decode_leb_128_array(bytes.fromhex(hexbytes), 1).tolist() == [v]
    # a tensor in the file: the 17 bytes of the tag, the byte count as u32, the values
    w = S.NNUEWriter.__new__(S.NNUEWriter)
    w.buf = bytearray()
    w.write_tensor(torch.tensor([63, 64, -64, -65, 32767, -32768], dtype=torch.int16), "leb128")
    assert bytes(w.buf) == b"COMPRESSED_LEB128" + bytes.fromhex("0c000000" "3f" "c000" "40" "bf7f" "ffff01" "80807e")


# What model/utils/serialize.py:102-160 and composed_feature_transformer.py:41-52 fix for a HalfKAv2_hm^ net, worked out
# by hand from those lines (nothing below calls this build's own hash functions):
#   feature hash 0x7F234CB8 (one feature block: rotate-left of 0, xor HASH); version 0x6A448AFA;
#   fc_hash: prev = 0xEC42E90D ^ 2 L1; per layer of out = L2, L3, 1 outputs: h = 0xCC03DAE4 + out, h ^= prev >> 1,
#   h ^= (prev << 31) mod 2^32, and + 0x538D24C7 mod 2^32 unless out == 1.
#     L1 = 1024: 0xEC42E10D -> 0x8DAFD049 -> 0x5E6157E7 -> 0x63337116       (L2 = 32, L3 = 32: the reference's defaults,
#     L1 = 3072: 0xEC42F10D -> 0x8DAFC739 -> 0x5E615D5F -> 0x6333744A        modules/config.py:10-15; L2 = 16: 15 + 1)
#   network hash = fc_hash ^ feature hash ^ 2 L1; feature transformer hash = feature hash ^ 2 L1.
#   Sections, uncompressed, behind the 84-byte default description (12 + 84 = 96): FT hash, int16 bias[L1],
#   int16 weight[22528, L1], int32 psqt[22528, 8], then per bucket: hash, int32 bias[L2], int8 [L2, L1], int32 bias[L3],
#   int8 [L3, 2 L2 padded to 32], int32 bias[1], int8 [1, 2 L2 + 2 L3 padded to 32].
LAYOUTS = [
    dict(L1=1024, L2=32, L3=32, header="fa8a446a" "ae35101c" "54000000", ft_hash=0x7F2344B8, fc_hash=0x63337116,
         ft_bias=100, ft_weight=2148, psqt=46139492, bucket0=46860388, bucket_bytes=35208,
         in_bucket=dict(l1_bias=4, l1_weight=132, l2_bias=32900, l2_weight=33028, out_bias=35076, out_weight=35080),
         size=47142052),
    dict(L1=3072, L2=16, L3=32, header="fa8a446a" "f220101c" "54000000", ft_hash=0x7F2354B8, fc_hash=0x6333744A,
         ft_bias=100, ft_weight=6244, psqt=138418276, bucket0=139139172, bucket_bytes=50472,
         in_bucket=dict(l1_bias=4, l1_weight=68, l2_bias=49220, l2_weight=49348, out_bias=50372, out_weight=50376),
         size=139542948),
]


@pytest.mark.parametrize("lay", LAYOUTS, ids=["default_1024_32_32", "config4_3072_16_32"])
def test_file_layout_against_literals_worked_out_from_the_reference(lay):
    L1, L2, L3 = lay["L1"], lay["L2"], lay["L3"]
    torch.manual_seed(L1)
    m = M.NNUEModel("HalfKAv2_hm^", M.ModelConfig(L1=L1, L2=L2, L3=L3))
    buf = bytes(S.NNUEWriter(m).buf)          # default description, no compression
    assert buf[:12].hex() == lay["header"]
    assert buf[12:96].decode() == "Network trained with the https://github.com/official-stockfish/nnue-pytorch trainer."
    assert struct.unpack_from("<I", buf, 96)[0] == lay["ft_hash"]
    assert len(buf) == lay["size"]
    for b in range(8):
        assert struct.unpack_from("<I", buf, lay["bucket0"] + b * lay["bucket_bytes"])[0] == lay["fc_hash"], b
    # every section at its literal offset holds the quantized tensor it is meant to
    export = m.input.get_export_weights()
    w16, b16, p32 = quantized.quantize_feature_transformer(export, m.input.bias.data, L1)
    assert np.array_equal(np.frombuffer(buf, "<i2", L1, lay["ft_bias"]), b16.numpy())
    for row in (0, 1, 22527):     # whole-table comparisons are the other test's; here the place of the rows
        assert np.array_equal(np.frombuffer(buf, "<i2", L1, lay["ft_weight"] + row * L1 * 2), w16[row].numpy())
        assert np.array_equal(np.frombuffer(buf, "<i4", 8, lay["psqt"] + row * 32), p32[row].numpy())
    w1, b1, w2, b2, wo, bo = [t.numpy() for t in quantized.quantize_layer_stacks(m.layer_stacks)]
    pad = lambda n: (n + 31) // 32 * 32
    for b in (0, 7):
        at = lay["bucket0"] + b * lay["bucket_bytes"]
        o = lay["in_bucket"]
        assert np.array_equal(np.frombuffer(buf, "<i4", L2, at + o["l1_bias"]), b1[b * L2:(b + 1) * L2])
        assert np.array_equal(np.frombuffer(buf, "i1", L2 * L1, at + o["l1_weight"]).reshape(L2, L1), w1[b * L2:(b + 1) * L2])
        assert np.array_equal(np.frombuffer(buf, "<i4", L3, at + o["l2_bias"]), b2[b * L3:(b + 1) * L3])
        l2w = np.frombuffer(buf, "i1", L3 * pad(2 * L2), at + o["l2_weight"]).reshape(L3, pad(2 * L2))
        assert np.array_equal(l2w[:, :2 * L2], w2[b * L3:(b + 1) * L3]) and not l2w[:, 2 * L2:].any()
        assert np.array_equal(np.frombuffer(buf, "<i4", 1, at + o["out_bias"]), bo[b:b + 1])
        ow = np.frombuffer(buf, "i1", pad(2 * L2 + 2 * L3), at + o["out_weight"])
        assert np.array_equal(ow[:2 * L2 + 2 * L3], wo[b]) and not ow[2 * L2 + 2 * L3:].any()
    # and the reader takes the file for exactly this architecture
    r = S.NNUEReader(io.BytesIO(buf), "HalfKAv2_hm^", M.ModelConfig(L1=L1, L2=L2, L3=L3))
    assert r.description.startswith("Network trained with")


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
