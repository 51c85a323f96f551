"""The checkpoint reader/writer (burn_dragon_amd/record.py) and the tokenizers against the data files
the reference ships under www/assets/model/tiny_shakespeare (copied as data into
tests/golden/tiny_shakespeare: model.bin, config.json, vocab.json), and the oracle on those trained
weights.

The trained checkpoint is the strongest pin the reference offers for the values of
forward_with_state: a restatement with a wrong sign, a dropped LayerNorm, a transposed weight or the
wrong positional scheme scores near the uniform loss ln(69) = 4.23 nats on Shakespeare text, the
right one near 1.2.
"""
import json
import os

import numpy as np
import pytest

from burn_dragon_amd import record
from burn_dragon_amd.positional import RotaryEmbedding
from burn_dragon_amd.tokenizer import ByteTokenizer, CharVocab
from oracle import bdh_oracle as orc

CKPT = os.path.join(os.path.dirname(__file__), "golden", "tiny_shakespeare")
TEXT = ("First Citizen:\nBefore we proceed any further, hear me speak.\n\nAll:\nSpeak, speak.\n\n"
        "First Citizen:\nYou are all resolved rather to die than to famish?\n\nAll:\nResolved. resolved.\n")


def test_shipped_record_parses():
    with open(os.path.join(CKPT, "model.bin"), "rb") as f:
        buf = f.read()
    meta, params = record.parse_record(buf)
    assert (meta.float, meta.int, meta.version, meta.settings) == ("f32", "i32", "0.19.1", "FullPrecisionSettings")
    assert "BinFileRecorder" in meta.format
    assert [p.shape for p in params] == [(69, 128), (4, 128, 128), (4, 128, 128), (512, 128), (128, 69)]
    assert all(p.dtype == "f32" and len(p.id) == 13 for p in params)
    assert sum(p.data.nbytes for p in params) == 857088  # everything but 256 bytes of framing is payload
    w = record.weights_from_params(params)
    assert record.infer_dimensions(w) == {"vocab_size": 69, "n_embd": 128, "n_head": 4, "mlp_internal_dim_multiplier": 4}
    assert all(np.isfinite(v).all() for v in w.values())


def test_checkpoint_dir_gives_the_reference_config():
    cfg, w, vocab, block_size = record.load_checkpoint_dir(CKPT)
    assert (cfg.n_layer, cfg.n_embd, cfg.n_head, cfg.mlp_internal_dim_multiplier, cfg.vocab_size) == (4, 128, 4, 4, 69)
    assert cfg.latent_per_head() == 128 and block_size == 512
    assert cfg.fused_kernels.enabled and cfg.fused_kernels.rotary_embedding == RotaryEmbedding.ALIBI
    assert cfg.fused_kernels.block_sparse.time.block_size == 512  # src/inference.rs:28-32
    assert len(CharVocab.from_json_str(vocab)) == 69


@pytest.mark.parametrize("half", [False, True])
def test_writer_round_trip(tmp_path, half):
    rng = np.random.default_rng(3)
    h, d, N, V = 2, 8, 16, 11
    w = {"embed": rng.standard_normal((V, d)), "encoder": rng.standard_normal((h, d, N)),
         "encoder_v": rng.standard_normal((h, d, N)), "decoder": rng.standard_normal((h * N, d)),
         "lm_head": rng.standard_normal((d, V))}
    w = {k: v.astype(np.float32) for k, v in w.items()}
    path = record.save_record(str(tmp_path / "model"), w, half=half)
    assert path.endswith("model.bin")
    meta, back = record.load_record(str(tmp_path / "model"))  # base name, as the recorder takes it
    assert meta.settings == ("HalfPrecisionSettings" if half else "FullPrecisionSettings")
    for k in w:
        if half:
            assert np.array_equal(back[k], w[k].astype(np.float16).astype(np.float32))
        else:
            assert np.array_equal(back[k], w[k])


def test_shipped_record_reserialises_to_the_same_parameters():
    _, w = record.load_record(os.path.join(CKPT, "model.bin"))
    meta, params = record.parse_record(record.serialize_record(w))
    assert meta.settings == "FullPrecisionSettings"
    for p, name in zip(params, record.PARAM_ORDER):
        assert np.array_equal(p.data, w[name])


def test_damaged_records_are_rejected():
    with open(os.path.join(CKPT, "model.bin"), "rb") as f:
        buf = f.read()
    with pytest.raises(record.RecordError):
        record.parse_record(buf[:5000])  # truncated inside the first tensor
    with pytest.raises(record.RecordError):
        record.parse_record(b"\x03abc" * 5 + buf[200:])  # not a recorder header
    meta, params = record.parse_record(buf)
    with pytest.raises(record.RecordError):
        record.weights_from_params(params[:4])
    swapped = [params[0], params[3], params[2], params[1], params[4]]
    with pytest.raises(record.RecordError):
        record.weights_from_params(swapped)
    bad = bytearray(buf)
    # the dtype index follows the shape of the first tensor: 152 header bytes + payload + rank + 2 dims
    off = 152 + 35328 + 3
    assert bad[off] == 1
    bad[off] = 9  # an integer dtype
    with pytest.raises(record.RecordError):
        record.parse_record(bytes(bad))


def _loss(corc, w, ids, rotary):
    shape = orc.BDHShape(n_layer=4, n_embd=128, n_head=4, mlp_internal_dim_multiplier=4, vocab_size=69, rotary=rotary)
    Nq = 128 * (2 if rotary == orc.POPE else 1)
    rho = np.zeros((4, 1, 4, Nq, 128), np.float32)
    logits, pos, x, _ = corc.forward_with_state(shape, orc.BDHWeights(**w), ids, rho, 0, taps=True, sparse_state=False)
    z = logits[0].astype(np.float64)
    logp = z - z.max(-1, keepdims=True)
    logp -= np.log(np.exp(logp).sum(-1, keepdims=True))
    return float(-logp[np.arange(ids.shape[1] - 1), ids[0, 1:]].mean()), logits, x


def test_oracle_predicts_shakespeare_with_the_trained_weights(corc):
    """Pins the values of the oracle's forward_with_state (ALiBi variant, which shares everything but
    the positional scheme with the others) on real trained weights."""
    _, w, vocab, _ = record.load_checkpoint_dir(CKPT)
    tok = CharVocab.from_json_str(vocab)
    ids = np.array([tok.encode(TEXT)])
    loss, logits, x = _loss(corc, w, ids, orc.ALIBI)
    assert loss < 1.35, loss  # measured 1.16; uniform = 4.23
    predicted = tok.decode([int(i) for i in logits[0].argmax(-1)])
    assert sum(a == b for a, b in zip(predicted[:-1], TEXT[1:])) > 0.6 * (len(TEXT) - 1)
    assert 0.2 < (x > 0).mean() < 0.5  # trained activations are sparser than the random-init half
    # sensitivity: the same weights under the wrong positional scheme are no better than uniform
    assert _loss(corc, w, ids, orc.ROPE)[0] > 3.5
    assert _loss(corc, w, ids, orc.POPE)[0] > 3.5
    # and so is a model whose two encoders are swapped
    swapped = dict(w, encoder=w["encoder_v"], encoder_v=w["encoder"])
    assert _loss(corc, swapped, ids, orc.ALIBI)[0] > 2.5


def test_numpy_oracle_agrees_on_the_trained_weights(corc):
    _, w, vocab, _ = record.load_checkpoint_dir(CKPT)
    ids = np.array([CharVocab.from_json_str(vocab).encode(TEXT[:40])])
    shape = orc.BDHShape(n_layer=4, n_embd=128, n_head=4, mlp_internal_dim_multiplier=4, vocab_size=69, rotary=orc.ALIBI)
    W = orc.BDHWeights(**w)
    rho = np.zeros((4, 1, 4, 128, 128), np.float32)
    logits_c, _, _, _ = corc.forward_with_state(shape, W, ids, rho, 0, sparse_state=False)
    logits_np = orc.forward_with_state(shape, W, ids, orc.ModelState(4))
    assert np.abs(logits_c - logits_np).max() < 1e-3 * np.abs(logits_np).max()


# ---- tokenizers: the reference's own tests (src/tokenizer/byte.rs:104-126, char_vocab.rs:281-314) ----
def test_byte_tokenizer_round_trip_and_eos():
    t = ByteTokenizer(True)
    enc = t.encode("hello", True, True)
    assert enc[0] == t.bos_id() == 256 and enc[-1] == t.eos_id() == 257 and t.pad_id() == 258 and len(t) == 259
    assert t.decode(enc) == "hello"
    ids = t.encode("abc", False, False) + [t.eos_id()] + [ord("d"), ord("e")]
    assert t.decode(ids) == "abc"
    plain = ByteTokenizer(False)
    assert len(plain) == 256 and plain.bos_id() is None and plain.encode("é", True, True) == [0xC3, 0xA9]
    assert plain.decode([0xC3, 0xA9, 300]) == "é"


def test_char_vocab_fit_encode_decode_unknown_and_save(tmp_path):
    vocab = CharVocab.fit(["hello", "world"], True)
    assert len(vocab) >= 4
    enc = vocab.encode("hello", True, True)
    assert enc[0] == vocab.bos_id() and enc[-1] == vocab.eos_id()
    assert vocab.decode(enc) == "hello"
    small = CharVocab.fit(["ab"], True)
    toks = small.encode("ac", False, False)
    assert toks == [small.ch2id["a"], small.unk_id()]
    assert small.decode(toks) == "a?"
    with pytest.raises(KeyError):
        CharVocab.fit(["ab"], False).encode("c")
    path = str(tmp_path / "vocab.json")
    vocab.save(path)
    assert CharVocab.load(path) == vocab


def test_shipped_vocabulary():
    with open(os.path.join(CKPT, "vocab.json"), "r", encoding="utf-8") as f:
        text = f.read()
    vocab = CharVocab.from_json_str(text)
    rec = json.loads(text)
    assert (vocab.pad_id(), vocab.bos_id(), vocab.eos_id(), vocab.unk_id()) == (0, 1, 2, 3) and len(vocab) == 69
    assert vocab.id2ch[4:9] == list("First")  # first-seen order of the corpus
    ids = vocab.encode(TEXT)
    assert vocab.decode(ids) == TEXT and max(ids) < 69
    assert vocab.to_record() == rec
