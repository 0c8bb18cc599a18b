"""Seq2SeqSharp model files: reader (and a writer, for tools and tests).

A model file is `ProtoBuf.Serializer.Serialize(stream, Model_4_ProtoBufSerializer)` (Seq2SeqSharp/Tools/BaseSeq2SeqFramework.cs:233,
contract in Seq2SeqSharp/Models/Model_4_ProtoBufSerializer.cs:243-324): plain protocol-buffer wire format, no container.
protobuf-net writes a Dictionary as a repeated message {1: key, 2: value}, arrays of numbers as repeated scalars (packed into
one length-delimited field or one field per element: a reader accepts both), enums and ints as varints (negative int32 as
the 64-bit two's complement), nested contracts as length-delimited messages.

    fields: 1 Name2Weights map<string, float[]>     2 DecoderEmbeddingDim   3 EncoderEmbeddingDim   4 DecoderLayerDepth
            5 EncoderLayerDepth  6 DecoderType  7 EncoderType  8 HiddenDim  9 IntermediateDim  10 EnableSegmentEmbeddings
            11 MultiHeadNum  12 SrcVocab  13 TgtVocab  14 ClsVocabs[]  15 EnableCoverageModel  16 SharedEmbeddings
            17 SimilarityType  18 EnableTagEmbeddings  19 MaxSegmentNum  20 PointerGenerator  21 ExpertNum
            22 ExpertsPerTokenFactor  23 ActivateFunc  24 VQType  25 Name2WeightsVQ map<string, bytes>
            26 Name2CodeBook map<string, double[]>  27 Name2WeightsHalf map<string, uint16[]>  28 PEType  29 NormType
            30 MultiHeadAttentionType  31 KVGroupNum
    vocabulary (fields 12-14): 1 map<string, int32> word -> index, 2 map<int32, string> index -> word, 3 IgnoreCase

Weights are stored four ways (Models/Model.cs:178-258, read back at :259-310): float32 (field 1), float16 bit patterns (27,
VQType FLOAT16 = 65536), and 256- or 16-entry vector quantisation (25 + 26, VQType INT8 = 256 / INT4 = 16: one byte per
weight, or two weights per byte with the LOW nibble first).

The reference ships no model file (its pretrained blobs are absent from the source tree), so this reader is checked against
the wire format itself: an independent encoder (google.protobuf) and hand-assembled bytes, not against a reference file.
"""
import struct

import numpy as np

# enum values of the reference (Utils/ModeEnums.cs:33-53, Utils/ActivateFuncEnums.cs:13-20, Utils/PositionEmbedding.cs:18-23,
# Utils/AttentionTypeEnums.cs:15-19)
DECODER_GPT = 2
VQ_NONE, VQ_FLOAT16, VQ_INT8, VQ_INT4 = 0, 65536, 256, 16
NORM_LAYERNORM, NORM_RMSNORM = 0, 1
PE_APE, PE_NOPE, PE_ROPE = 0, 1, 2
MHA, GQA = 0, 1

_INT_FIELDS = {2: "DecoderEmbeddingDim", 3: "EncoderEmbeddingDim", 4: "DecoderLayerDepth", 5: "EncoderLayerDepth", 6: "DecoderType",
               7: "EncoderType", 8: "HiddenDim", 9: "IntermediateDim", 10: "EnableSegmentEmbeddings", 11: "MultiHeadNum",
               15: "EnableCoverageModel", 16: "SharedEmbeddings", 18: "EnableTagEmbeddings", 19: "MaxSegmentNum", 20: "PointerGenerator",
               21: "ExpertNum", 22: "ExpertsPerTokenFactor", 23: "ActivateFunc", 24: "VQType", 28: "PEType", 29: "NormType",
               30: "MultiHeadAttentionType", 31: "KVGroupNum"}


# ---- wire format -------------------------------------------------------------------------------
def _varint(buf, pos):
    out, shift = 0, 0
    while True:
        b = buf[pos]
        pos += 1
        out |= (b & 0x7F) << shift
        if not b & 0x80:
            return out, pos
        shift += 7
        if shift > 70:
            raise ValueError("model file: varint longer than ten bytes")


def _int32(v):
    """A varint read as int32 / int64 in two's complement."""
    v &= (1 << 64) - 1
    return v - (1 << 64) if v >> 63 else v


def _fields(buf, start=0, end=None):
    """Yield (field number, wire type, value) over one message; value is an int (varint, fixed) or a memoryview (length-delimited)."""
    pos = start
    end = len(buf) if end is None else end
    while pos < end:
        tag, pos = _varint(buf, pos)
        field, wt = tag >> 3, tag & 7
        if wt == 0:
            v, pos = _varint(buf, pos)
        elif wt == 1:
            v = struct.unpack_from("<Q", buf, pos)[0]
            pos += 8
        elif wt == 2:
            n, pos = _varint(buf, pos)
            if pos + n > end:
                raise ValueError("model file: a field runs past the end of its message")
            v = buf[pos:pos + n]
            pos += n
        elif wt == 5:
            v = struct.unpack_from("<I", buf, pos)[0]
            pos += 4
        else:
            raise ValueError("model file: unsupported wire type %d" % wt)
        yield field, wt, v
    if pos != end:
        raise ValueError("model file: message length mismatch")


def _repeated(chunks, fixed_dtype):
    """A repeated number field from its occurrences [(wire type, value)]: packed blocks and single elements, in file order.
    fixed_dtype: '<f4' / '<f8' for fixed-width elements, None for varints."""
    parts = []
    for wt, v in chunks:
        if wt == 2:
            if fixed_dtype:
                parts.append(np.frombuffer(v, dtype=fixed_dtype))
            else:
                vals, pos = [], 0
                while pos < len(v):
                    x, pos = _varint(v, pos)
                    vals.append(x)
                parts.append(np.array(vals, np.uint64))
        elif fixed_dtype:
            parts.append(np.array([v], "<u4" if fixed_dtype == "<f4" else "<u8").view(fixed_dtype))
        else:
            parts.append(np.array([v], np.uint64))
    if not parts:
        return np.zeros((0,), fixed_dtype or np.uint64)
    return np.concatenate(parts)


def _map_entries(entry_views):
    for ev in entry_views:
        key, vals = None, []
        for f, wt, v in _fields(ev):
            if f == 1:
                key = (wt, v)
            elif f == 2:
                vals.append((wt, v))
        yield key, vals


def _read_vocab(view):
    w2i, i2w, ignore = {}, {}, False
    f1, f2 = [], []
    for f, wt, v in _fields(view):
        if f == 1:
            f1.append(v)
        elif f == 2:
            f2.append(v)
        elif f == 3:
            ignore = bool(v)
    for key, vals in _map_entries(f1):
        w2i[bytes(key[1]).decode("utf-8") if key else ""] = _int32(vals[-1][1]) if vals else 0
    for key, vals in _map_entries(f2):
        i2w[_int32(key[1]) if key else 0] = bytes(vals[-1][1]).decode("utf-8") if vals else ""
    return {"word_to_index": w2i, "index_to_word": i2w, "ignore_case": ignore}


def read_model(path_or_bytes):
    """Parse a model file.  Returns a dict: the scalar fields by their C# names, 'SrcVocab' / 'TgtVocab' / 'ClsVocabs',
    and the four weight dictionaries as stored ('Name2Weights' float32, 'Name2WeightsHalf' uint16, 'Name2WeightsVQ' uint8,
    'Name2CodeBook' float64)."""
    buf = path_or_bytes if isinstance(path_or_bytes, (bytes, bytearray, memoryview)) else open(path_or_bytes, "rb").read()
    buf = memoryview(bytes(buf))
    m = {name: 0 for name in _INT_FIELDS.values()}
    m.update(SimilarityType=None, SrcVocab=None, TgtVocab=None, ClsVocabs=[], Name2Weights={}, Name2WeightsHalf={}, Name2WeightsVQ={}, Name2CodeBook={})
    maps = {1: [], 25: [], 26: [], 27: []}
    for f, wt, v in _fields(buf):
        if f in _INT_FIELDS:
            m[_INT_FIELDS[f]] = _int32(v)
        elif f in maps:
            maps[f].append(v)
        elif f == 12:
            m["SrcVocab"] = _read_vocab(v)
        elif f == 13:
            m["TgtVocab"] = _read_vocab(v)
        elif f == 14:
            m["ClsVocabs"].append(_read_vocab(v))
        elif f == 17:
            m["SimilarityType"] = bytes(v).decode("utf-8")
        # unknown fields are skipped, as protobuf readers do
    for key, vals in _map_entries(maps[1]):
        m["Name2Weights"][bytes(key[1]).decode("utf-8")] = _repeated(vals, "<f4").astype(np.float32)
    for key, vals in _map_entries(maps[27]):
        m["Name2WeightsHalf"][bytes(key[1]).decode("utf-8")] = _repeated(vals, None).astype(np.uint16)
    for key, vals in _map_entries(maps[25]):
        m["Name2WeightsVQ"][bytes(key[1]).decode("utf-8")] = np.frombuffer(b"".join(bytes(v) for _, v in vals), np.uint8)
    for key, vals in _map_entries(maps[26]):
        m["Name2CodeBook"][bytes(key[1]).decode("utf-8")] = _repeated(vals, "<f8").astype(np.float64)
    return m


def get_weights(m, name):
    """Model.GetWeights (Models/Model.cs:259-310) / GetWeightsHalfType: the float32 values of one parameter, whatever way it is
    stored.  Float16 patterns convert exactly; quantised weights go through their code book (INT4: low nibble first)."""
    if name in m["Name2Weights"]:
        return m["Name2Weights"][name]
    if name in m["Name2WeightsHalf"]:
        return m["Name2WeightsHalf"][name].view(np.float16).astype(np.float32)
    if name in m["Name2WeightsVQ"]:
        book, q = m["Name2CodeBook"][name], m["Name2WeightsVQ"][name]
        if m["VQType"] == VQ_INT8:
            return book[q].astype(np.float32)
        if m["VQType"] == VQ_INT4:
            out = np.empty((q.size * 2,), np.float32)
            out[0::2] = book[q & 0x0F]
            out[1::2] = book[q >> 4]
            return out
    raise KeyError("weight '%s' doesn't exist in the model" % name)


def gpt_config(m, dtype=None):
    """The GPTDecoder configuration (seq2seqsharp_amd.synth's dict form) of a model file written by the reference's GPT task."""
    from . import synth
    if m["DecoderType"] != DECODER_GPT:
        raise ValueError("model file: DecoderType %d is not GPTDecoder" % m["DecoderType"])
    if m["PEType"] == PE_APE:
        raise ValueError("model file: absolute position embeddings (PEType APE) are outside the decode path built here (RoPE and NoPE are supported)")
    max_segments, sep_id = 0, 3
    if m["EnableSegmentEmbeddings"]:
        # CreateTokensEmbeddings adds SegmentEmbedding[segment index] to every token embedding (Utils/TensorUtils.cs:147-152,
        # table [MaxSegmentNum, EncoderEmbeddingDim] built by Misc.CreateAuxEmbeddings, Utils/Misc.cs:164-168); the segment index
        # counts the vocabulary's "[SEP]" tokens (BuildInTokens.SEP)
        max_segments = m["MaxSegmentNum"]
        if max_segments < 1:
            raise ValueError("model file: EnableSegmentEmbeddings with MaxSegmentNum %d" % max_segments)
        if m["EncoderEmbeddingDim"] and m["EncoderEmbeddingDim"] != m["HiddenDim"]:
            raise ValueError("model file: the segment embedding table is %d wide, the decoder's hidden size is %d" % (m["EncoderEmbeddingDim"], m["HiddenDim"]))
        words = m["TgtVocab"]["word_to_index"] if m["TgtVocab"] else {}
        if "[SEP]" not in words:
            raise ValueError("model file: segment embeddings are enabled but the target vocabulary has no [SEP] token")
        sep_id = int(words["[SEP]"])
    # EnableTagEmbeddings does not change GPTDecoder's results: Decoder.GPTDecode calls CreateTokensEmbeddings without
    # enableTagEmbedding (Applications/Decoder.cs:673,695; only Encoder.cs:102 passes it), so the flag is accepted
    vocab = len(m["TgtVocab"]["index_to_word"]) if m["TgtVocab"] else 0
    heads = m["MultiHeadNum"]
    gqa = m["MultiHeadAttentionType"] == GQA
    if dtype is None:
        dtype = "f16" if m["VQType"] == VQ_FLOAT16 else "f32"
    return dict(n_layers=m["DecoderLayerDepth"], hidden=m["HiddenDim"], n_heads=heads, n_kv_heads=m["KVGroupNum"] if gqa else heads,
                ffn_dim=m["IntermediateDim"], vocab=vocab, attn_type=synth.GQA if gqa else synth.MHA,
                norm_type=synth.RMSNORM if m["NormType"] == NORM_RMSNORM else synth.LAYERNORM, act=m["ActivateFunc"],
                n_experts=max(m["ExpertNum"], 1), experts_per_token=max(m["ExpertsPerTokenFactor"], 1), norm_eps=1e-6, rope_base=500000.0,
                use_rope=1 if m["PEType"] == PE_ROPE else 0, dtype=dtype, max_segments=max_segments, sep_token_id=sep_id)


def load_gpt(path_or_bytes, dtype=None):
    """Model file -> (config dict, {parameter name: float32 array in its saved shape}, target vocabulary).  The weights feed
    seq2seqsharp_amd.gpt.HipGpt (TSHip_GptSetWeight) as they are."""
    from . import synth
    m = read_model(path_or_bytes)
    cfg = gpt_config(m, dtype)
    weights = {}
    for name, shape, _ in synth.weight_shapes(cfg):
        flat = get_weights(m, name)
        if flat.size != int(np.prod(shape)):
            raise ValueError("model file: weight '%s' holds %d values, the configuration needs %s" % (name, flat.size, list(shape)))
        weights[name] = flat.reshape(shape)
    # a parameter in the file that the decode path would not consume (a segment or position embedding table, another
    # network's layers) means the file describes a model this path does not compute: refuse rather than ignore it
    stored = set(m["Name2Weights"]) | set(m["Name2WeightsHalf"]) | set(m["Name2WeightsVQ"])
    extra = sorted(stored - set(weights))
    if extra:
        raise ValueError("model file: %d parameter(s) that the GPTDecoder path does not use: %s" % (len(extra), ", ".join(extra[:8])))
    return cfg, weights, m["TgtVocab"]


# ---- writer ------------------------------------------------------------------------------------
def _enc_varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def _tag(field, wt):
    return _enc_varint((field << 3) | wt)


def _ld(field, payload):
    return _tag(field, 2) + _enc_varint(len(payload)) + payload


def _write_vocab(v):
    out = b""
    for w, i in v["word_to_index"].items():
        out += _ld(1, _ld(1, w.encode("utf-8")) + _tag(2, 0) + _enc_varint(i))
    for i, w in v["index_to_word"].items():
        out += _ld(2, _tag(1, 0) + _enc_varint(i) + _ld(2, w.encode("utf-8")))
    if v.get("ignore_case"):
        out += _tag(3, 0) + _enc_varint(1)
    return out


def write_model(m, packed=True):
    """Serialise a dict in read_model's form.  packed=False writes one field per array element (the other encoding a reader
    must accept).  Zero / false / empty members are left out, as protobuf-net leaves out defaults."""
    out = b""

    def arr(field, a, kind):
        a = np.asarray(a)
        if kind == "f4":
            raw = a.astype("<f4")
            return _ld(field, raw.tobytes()) if packed else b"".join(_tag(field, 5) + raw[i:i + 1].tobytes() for i in range(raw.size))
        if kind == "f8":
            raw = a.astype("<f8")
            return _ld(field, raw.tobytes()) if packed else b"".join(_tag(field, 1) + raw[i:i + 1].tobytes() for i in range(raw.size))
        enc = [_enc_varint(int(x)) for x in a]
        return _ld(field, b"".join(enc)) if packed else b"".join(_tag(field, 0) + e for e in enc)

    for name, w in m.get("Name2Weights", {}).items():
        out += _ld(1, _ld(1, name.encode("utf-8")) + arr(2, w, "f4"))
    for f in sorted(_INT_FIELDS):
        if f < 12 and m.get(_INT_FIELDS[f], 0):
            out += _tag(f, 0) + _enc_varint(int(m[_INT_FIELDS[f]]))
    if m.get("SrcVocab"):
        out += _ld(12, _write_vocab(m["SrcVocab"]))
    if m.get("TgtVocab"):
        out += _ld(13, _write_vocab(m["TgtVocab"]))
    for v in m.get("ClsVocabs", []):
        out += _ld(14, _write_vocab(v))
    for f in sorted(_INT_FIELDS):
        if 12 < f < 25 and m.get(_INT_FIELDS[f], 0):
            out += _tag(f, 0) + _enc_varint(int(m[_INT_FIELDS[f]]))
        if f == 16 and m.get("SimilarityType") is not None:
            out += _ld(17, m["SimilarityType"].encode("utf-8"))
    for name, q in m.get("Name2WeightsVQ", {}).items():
        out += _ld(25, _ld(1, name.encode("utf-8")) + _ld(2, np.asarray(q, np.uint8).tobytes()))
    for name, b in m.get("Name2CodeBook", {}).items():
        out += _ld(26, _ld(1, name.encode("utf-8")) + arr(2, b, "f8"))
    for name, hbits in m.get("Name2WeightsHalf", {}).items():
        out += _ld(27, _ld(1, name.encode("utf-8")) + arr(2, hbits, "varint"))
    for f in sorted(_INT_FIELDS):
        if f > 27 and m.get(_INT_FIELDS[f], 0):
            out += _tag(f, 0) + _enc_varint(int(m[_INT_FIELDS[f]]))
    return out


def save_gpt(cfg, weights, path=None, storage="f32", vocab_words=None):
    """Write a GPTDecoder model the way Model.AddWeights stores it (Models/Model.cs:178-258): storage 'f32', 'f16' (VQType
    FLOAT16) or 'int8' (256-entry code book per tensor: here the code book is the sorted unique values when there are at most
    256 of them, else a uniform grid).  Returns the bytes (and writes them to `path` when given)."""
    from . import synth
    V = cfg["vocab"]
    words = vocab_words or ["</s>", "<s>", "<unk>", "[SEP]", "[CLS]"] + ["w%d" % i for i in range(5, V)]
    vocab = {"word_to_index": {w: i for i, w in enumerate(words[:V])}, "index_to_word": {i: w for i, w in enumerate(words[:V])}, "ignore_case": False}
    m = dict(DecoderEmbeddingDim=cfg["hidden"], DecoderLayerDepth=cfg["n_layers"], DecoderType=DECODER_GPT, EncoderType=-1, HiddenDim=cfg["hidden"],
             IntermediateDim=cfg["ffn_dim"], MultiHeadNum=cfg["n_heads"], TgtVocab=vocab, SrcVocab=vocab, ExpertNum=cfg.get("n_experts", 1),
             ExpertsPerTokenFactor=cfg.get("experts_per_token", 1), ActivateFunc=cfg["act"],
             VQType={"f32": VQ_NONE, "f16": VQ_FLOAT16, "int8": VQ_INT8}[storage], PEType=PE_ROPE if cfg.get("use_rope", 1) else PE_NOPE,
             NormType=NORM_RMSNORM if cfg["norm_type"] == synth.RMSNORM else NORM_LAYERNORM,
             MultiHeadAttentionType=GQA if cfg["attn_type"] == synth.GQA else MHA, KVGroupNum=cfg["n_kv_heads"] if cfg["attn_type"] == synth.GQA else 0,
             Name2Weights={}, Name2WeightsHalf={}, Name2WeightsVQ={}, Name2CodeBook={})
    if cfg.get("max_segments", 0) > 0:
        m.update(EnableSegmentEmbeddings=1, MaxSegmentNum=cfg["max_segments"], EncoderEmbeddingDim=cfg["hidden"])
    for name, w in weights.items():
        flat = np.asarray(w, np.float32).reshape(-1)
        if storage == "f32":
            m["Name2Weights"][name] = flat
        elif storage == "f16":
            m["Name2WeightsHalf"][name] = flat.astype(np.float16).view(np.uint16)
        else:
            uniq = np.unique(flat)
            book = uniq if uniq.size <= 256 else np.linspace(flat.min(), flat.max(), 256)
            book = np.concatenate([book, np.zeros(256 - book.size)]).astype(np.float64)
            m["Name2CodeBook"][name] = book
            m["Name2WeightsVQ"][name] = np.abs(flat[:, None].astype(np.float64) - book[None, :]).argmin(1).astype(np.uint8) if flat.size * 256 < 5e7 \
                else np.searchsorted((book[1:] + book[:-1]) / 2, flat).astype(np.uint8)
    data = write_model(m)
    if path:
        with open(path, "wb") as f:
            f.write(data)
    return data
