"""Model files (Models/Model_4_ProtoBufSerializer.cs:243-324 written with protobuf-net, Tools/BaseSeq2SeqFramework.cs:233): the
reader is checked against the wire format itself -- known-answer bytes of the protocol-buffer encoding guide and an
independent encoder/decoder (google.protobuf with a schema built here from the contract's field numbers) -- because the
reference's source tree holds no model file to read."""
import numpy as np
import pytest

from seq2seqsharp_amd import model_file as mf
from seq2seqsharp_amd import synth


def test_wire_format_known_answers():
    # the encoding guide's examples: 150 in field 1; "testing" in field 2; packed [3, 270, 86942] in field 4
    assert mf._tag(1, 0) + mf._enc_varint(150) == bytes.fromhex("089601")
    assert mf._ld(2, b"testing") == bytes.fromhex("120774657374696e67")
    got = list(mf._fields(memoryview(bytes.fromhex("089601" "120774657374696e67" "2206038e029ea705"))))
    assert got[0] == (1, 0, 150) and bytes(got[1][2]) == b"testing" and got[2][0] == 4
    assert mf._repeated([(2, got[2][2])], None).tolist() == [3, 270, 86942]
    # a negative int32 is ten bytes of 64-bit two's complement
    assert mf._enc_varint(-1) == b"\xff" * 9 + b"\x01" and mf._int32(mf._varint(mf._enc_varint(-2), 0)[0]) == -2
    # packed and one-field-per-element forms of the same float array, mixed in one message
    a = np.array([1.5, -2.25, 3e-8], "<f4")
    chunks = [(5, int(a[:1].view("<u4")[0])), (2, memoryview(a[1:].tobytes()))]
    assert np.array_equal(mf._repeated(chunks, "<f4"), a)
    with pytest.raises(ValueError):
        list(mf._fields(memoryview(b"\x12\x09abc")))            # length runs past the end


def _schema():
    """The contract as a google.protobuf schema: dictionaries are repeated {1: key, 2: value} messages."""
    from google.protobuf import descriptor_pb2, descriptor_pool, message_factory
    F = descriptor_pb2.FieldDescriptorProto
    fd = descriptor_pb2.FileDescriptorProto(name="s2s_model_test.proto", package="s2stest", syntax="proto2")

    def msg(name, fields):
        m = fd.message_type.add(name=name)
        for fname, num, typ, label, tname, packed in fields:
            f = m.field.add(name=fname, number=num, type=typ, label=label)
            if tname:
                f.type_name = ".s2stest." + tname
            if packed is not None:
                f.options.packed = packed
    O, R = F.LABEL_OPTIONAL, F.LABEL_REPEATED
    for suffix, packed in (("P", True), ("U", False)):
        msg("WF" + suffix, [("key", 1, F.TYPE_STRING, O, None, None), ("value", 2, F.TYPE_FLOAT, R, None, packed)])
        msg("WH" + suffix, [("key", 1, F.TYPE_STRING, O, None, None), ("value", 2, F.TYPE_UINT32, R, None, packed)])
        msg("WD" + suffix, [("key", 1, F.TYPE_STRING, O, None, None), ("value", 2, F.TYPE_DOUBLE, R, None, packed)])
    msg("WB", [("key", 1, F.TYPE_STRING, O, None, None), ("value", 2, F.TYPE_BYTES, O, None, None)])
    msg("W2I", [("key", 1, F.TYPE_STRING, O, None, None), ("value", 2, F.TYPE_INT32, O, None, None)])
    msg("I2W", [("key", 1, F.TYPE_INT32, O, None, None), ("value", 2, F.TYPE_STRING, O, None, None)])
    msg("Vocab", [("w2i", 1, F.TYPE_MESSAGE, R, "W2I", None), ("i2w", 2, F.TYPE_MESSAGE, R, "I2W", None), ("ignore", 3, F.TYPE_BOOL, O, None, None)])
    ints = {n: num for num, n in mf._INT_FIELDS.items()}
    for suffix in ("P", "U"):
        fields = [("Name2Weights", 1, F.TYPE_MESSAGE, R, "WF" + suffix, None), ("SrcVocab", 12, F.TYPE_MESSAGE, O, "Vocab", None),
                  ("TgtVocab", 13, F.TYPE_MESSAGE, O, "Vocab", None), ("ClsVocabs", 14, F.TYPE_MESSAGE, R, "Vocab", None),
                  ("SimilarityType", 17, F.TYPE_STRING, O, None, None), ("Name2WeightsVQ", 25, F.TYPE_MESSAGE, R, "WB", None),
                  ("Name2CodeBook", 26, F.TYPE_MESSAGE, R, "WD" + suffix, None), ("Name2WeightsHalf", 27, F.TYPE_MESSAGE, R, "WH" + suffix, None)]
        for n, num in ints.items():
            fields.append((n, num, F.TYPE_BOOL if n in ("EnableSegmentEmbeddings", "EnableCoverageModel", "SharedEmbeddings", "EnableTagEmbeddings", "PointerGenerator")
                           else F.TYPE_INT32, O, None, None))
        msg("Model" + suffix, fields)
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    return {s: message_factory.GetMessageClass(pool.FindMessageTypeByName("s2stest.Model" + s)) for s in ("P", "U")}


@pytest.mark.parametrize("suffix", ["P", "U"])
def test_reader_against_an_independent_encoder(suffix):
    Model = _schema()[suffix]
    rng = np.random.default_rng(3)
    m = Model(DecoderEmbeddingDim=64, EncoderEmbeddingDim=0, DecoderLayerDepth=2, DecoderType=2, EncoderType=-1, HiddenDim=64, IntermediateDim=128,
              MultiHeadNum=4, SharedEmbeddings=True, ExpertNum=8, ExpertsPerTokenFactor=2, ActivateFunc=3, VQType=65536, PEType=2, NormType=1,
              MultiHeadAttentionType=1, KVGroupNum=2, SimilarityType="Continuous")
    wf = {"GPTDecoder.SelfAttn_0.m_Q": rng.standard_normal(37).astype(np.float32), "bias": np.array([0.0, -0.0, 1e-40, np.inf], np.float32)}
    for k, v in wf.items():
        e = m.Name2Weights.add(key=k)
        e.value.extend(v.tolist())
    wh = {"TgtEmbeddings": rng.integers(0, 65536, 50).astype(np.uint16)}
    for k, v in wh.items():
        m.Name2WeightsHalf.add(key=k).value.extend(v.tolist())
    m.Name2WeightsVQ.add(key="q", value=bytes(range(256)))
    m.Name2CodeBook.add(key="q").value.extend(np.linspace(-1, 1, 256).tolist())
    for i, w in enumerate(["</s>", "<s>", "<unk>", "naïve", "日本"]):
        m.TgtVocab.w2i.add(key=w, value=i)
        m.TgtVocab.i2w.add(key=i, value=w)
    m.TgtVocab.ignore = True
    m.ClsVocabs.add().w2i.add(key="a", value=7)
    got = mf.read_model(m.SerializeToString())
    assert got["EncoderType"] == -1 and got["VQType"] == mf.VQ_FLOAT16 and got["KVGroupNum"] == 2 and got["SharedEmbeddings"] == 1
    assert got["ExpertNum"] == 8 and got["ExpertsPerTokenFactor"] == 2 and got["SimilarityType"] == "Continuous" and got["EncoderEmbeddingDim"] == 0
    for k, v in wf.items():
        assert np.array_equal(got["Name2Weights"][k].view(np.uint32), v.view(np.uint32))          # bit patterns, -0.0 and denormals included
    assert np.array_equal(got["Name2WeightsHalf"]["TgtEmbeddings"], wh["TgtEmbeddings"])
    assert got["Name2WeightsVQ"]["q"].tolist() == list(range(256))
    assert np.array_equal(got["Name2CodeBook"]["q"], np.linspace(-1, 1, 256))
    assert got["TgtVocab"]["index_to_word"] == {0: "</s>", 1: "<s>", 2: "<unk>", 3: "naïve", 4: "日本"} and got["TgtVocab"]["ignore_case"]
    assert got["TgtVocab"]["word_to_index"]["日本"] == 4 and got["ClsVocabs"][0]["word_to_index"] == {"a": 7}
    assert got["SrcVocab"] is None


@pytest.mark.parametrize("packed", [True, False])
def test_writer_against_an_independent_decoder(packed):
    cfg = synth.tiny_config(n_experts=1)
    w = synth.make_weights(cfg, 2)
    m = mf.read_model(mf.save_gpt(cfg, w, storage="f32"))
    m["EncoderType"] = -1
    data = mf.write_model(m, packed=packed)
    pm = _schema()["P" if packed else "U"]()
    pm.ParseFromString(data)
    assert pm.EncoderType == -1 and pm.DecoderType == 2 and pm.HiddenDim == cfg["hidden"] and pm.KVGroupNum == cfg["n_kv_heads"]
    assert {e.key: e.value for e in pm.TgtVocab.i2w}[5] == "w5" and len(pm.TgtVocab.w2i) == cfg["vocab"]
    back = {e.key: np.array(e.value, np.float32) for e in pm.Name2Weights}
    assert set(back) == set(w)
    for k in w:
        assert np.array_equal(back[k], np.asarray(w[k], np.float32).reshape(-1))
    assert pm.SerializeToString() == data or not packed          # same bytes where the encoder has no freedom left


def test_stored_weight_forms():
    """Model.GetWeights (Models/Model.cs:259-310): float32 as is; Float16 bit patterns widen exactly; INT8 is one code-book index
    per weight; INT4 two per byte with the first weight of a pair in the low four bits (Model.cs:236-242 stores
    `highWeight * 16 + lowWeight`)."""
    book = np.zeros(256)
    book[:16] = np.arange(16) * 0.5 - 3
    m = dict(VQType=mf.VQ_INT4, Name2Weights={"a": np.array([1, 2], np.float32)}, Name2WeightsHalf={"h": np.array([0x3C00, 0xC000, 0x0001, 0x7BFF], np.uint16)},
             Name2WeightsVQ={"q": np.array([0x21, 0xF0], np.uint8)}, Name2CodeBook={"q": book})
    assert mf.get_weights(m, "a").tolist() == [1, 2]
    assert mf.get_weights(m, "h").tolist() == [1.0, -2.0, 2.0 ** -24, 65504.0]
    assert mf.get_weights(m, "q").tolist() == [book[1], book[2], book[0], book[15]]
    m["VQType"] = mf.VQ_INT8
    m["Name2WeightsVQ"]["q"] = np.array([15, 0, 3], np.uint8)
    assert mf.get_weights(m, "q").tolist() == [book[15], book[0], book[3]]
    with pytest.raises(KeyError):
        mf.get_weights(m, "missing")


@pytest.mark.parametrize("storage", ["f32", "f16", "int8"])
@pytest.mark.parametrize("kw", [dict(), dict(attn_type=synth.MHA, n_kv_heads=4, norm_type=synth.LAYERNORM, act=synth.RELU),
                                dict(n_experts=4, experts_per_token=2, norm_type=synth.LAYERNORM, act=synth.RELU, use_rope=0)])
def test_gpt_round_trip(storage, kw, tmp_path):
    cfg = synth.tiny_config(**kw)
    w = synth.make_weights(cfg, 4, random_bias=True)
    if storage == "int8":        # at most 256 distinct values per tensor, so that the code book is exact
        w = {k: (np.round(np.asarray(v) * 2000).clip(-120, 120) / 2000).astype(np.float32) for k, v in w.items()}
    path = tmp_path / "model.bin"
    mf.save_gpt(cfg, w, str(path), storage=storage)
    cfg2, w2, vocab = mf.load_gpt(str(path))
    for k in ("n_layers", "hidden", "n_heads", "n_kv_heads", "ffn_dim", "vocab", "attn_type", "norm_type", "act", "n_experts", "experts_per_token", "use_rope"):
        assert cfg2[k] == cfg[k], k
    assert cfg2["dtype"] == ("f16" if storage == "f16" else "f32") and cfg2["rope_base"] == 500000.0
    assert set(w2) == set(w) and vocab["index_to_word"][0] == "</s>"
    for k, v in w.items():
        v = np.asarray(v, np.float32)
        want = v.astype(np.float16).astype(np.float32) if storage == "f16" else v
        assert w2[k].shape == v.shape and np.array_equal(w2[k], want), k


def test_loader_refuses_what_the_path_does_not_cover():
    cfg = synth.tiny_config()
    m = mf.read_model(mf.save_gpt(cfg, synth.make_weights(cfg, 1)))
    m["DecoderType"] = 1
    with pytest.raises(ValueError, match="not GPTDecoder"):
        mf.load_gpt(mf.write_model(m))
    m["DecoderType"], m["PEType"] = mf.DECODER_GPT, mf.PE_APE
    with pytest.raises(ValueError, match="position"):
        mf.load_gpt(mf.write_model(m))
    m["PEType"] = mf.PE_ROPE
    m["Name2Weights"]["TgtEmbeddings"] = m["Name2Weights"]["TgtEmbeddings"][:-1]
    with pytest.raises(ValueError, match="holds"):
        mf.load_gpt(mf.write_model(m))


def test_loader_segment_embeddings_and_unused_parameters():
    """A file whose reference decode adds segment embeddings (Utils/TensorUtils.cs:147-152) loads with its table and its
    separator id, or not at all; one that stores parameters the path would ignore must not load silently.
    EnableTagEmbeddings is accepted: GPTDecode never passes it on."""
    cfg = synth.tiny_config()
    blob = mf.save_gpt(cfg, synth.make_weights(cfg, 1))
    m = mf.read_model(blob)
    m["EnableSegmentEmbeddings"], m["MaxSegmentNum"] = 1, 16      # the flag without the table: the table is then a missing weight
    with pytest.raises(KeyError, match="SegmentEmbedding"):
        mf.load_gpt(mf.write_model(m))
    m["MaxSegmentNum"] = 0
    with pytest.raises(ValueError, match="MaxSegmentNum"):
        mf.gpt_config(m)
    # with the table and a [SEP] word the model loads, and the configuration carries the table's height and the separator's id
    cfg_s = synth.tiny_config(max_segments=5)
    cfg2, w2, vocab = mf.load_gpt(mf.save_gpt(cfg_s, synth.make_weights(cfg_s, 2)))
    assert cfg2["max_segments"] == 5 and cfg2["sep_token_id"] == vocab["word_to_index"]["[SEP]"] == 3
    assert w2["SegmentEmbedding"].shape == (5, cfg_s["hidden"])
    m = mf.read_model(mf.save_gpt(cfg_s, synth.make_weights(cfg_s, 2), vocab_words=["</s>", "<s>", "<unk>"] + ["w%d" % i for i in range(3, cfg_s["vocab"])]))
    with pytest.raises(ValueError, match=r"no \[SEP\] token"):
        mf.gpt_config(m)
    m = mf.read_model(blob)
    m["MaxSegmentNum"] = 16          # the number alone changes nothing in the reference either
    m["EnableTagEmbeddings"] = 1
    cfg2, w2, _ = mf.load_gpt(mf.write_model(m))
    assert cfg2["hidden"] == cfg["hidden"] and "TgtEmbeddings" in w2
    for extra in ("SegmentEmbedding", "PosEmbedding", "GPTDecoder.SelfAttn_99.W0"):
        m = mf.read_model(blob)
        m["Name2Weights"][extra] = np.zeros((16 * cfg["hidden"],), np.float32)
        with pytest.raises(ValueError, match="does not use.*" + extra.replace(".", r"\.")):
            mf.load_gpt(mf.write_model(m))


def test_oracle_runs_a_loaded_model(oracle, tmp_path):
    """A model written as Float16, read back and fed to the oracle gives the logits of the fp16-rounded weights."""
    cfg = synth.tiny_config()
    w = synth.make_weights(cfg, 9)
    cfg2, w2, _ = mf.load_gpt(mf.save_gpt(cfg, w, storage="f16"), dtype="f32")
    cfg2.update(batch=cfg["batch"], prompt=cfg["prompt"], steps=cfg["steps"])
    ids = synth.make_prompts(cfg, 3)
    _, lg = oracle.OracleGpt(cfg2, w2).step(ids, use_cache=True)
    w16 = {k: np.asarray(v, np.float32).astype(np.float16).astype(np.float32) for k, v in w.items()}
    _, want = oracle.OracleGpt(dict(cfg, dtype="f32"), w16).step(ids, use_cache=True)
    assert np.array_equal(lg, want)
