"""The reference's tokenizer (Noeda/rllama src/tokenizer.rs): model-file parsing against the sentencepiece package on a
model trained here, the matching rules against expectations worked out by hand on a hand-built vocabulary, and the
C++ host mirror against the Python one.  CPU only."""
import io
import struct
import subprocess

import numpy as np
import pytest

from rllama_amd.tokenizer import Tokenizer, TokenizerError


def _vi(v):
    out = bytearray()
    while True:
        c = v & 0x7F
        v >>= 7
        out.append(c | (0x80 if v else 0))
        if not v:
            return bytes(out)


def _piece(piece=None, score=None, tp=None, extra=b""):
    m = b""
    if piece is not None:
        b = piece.encode("utf-8") if isinstance(piece, str) else piece
        m += b"\x0a" + _vi(len(b)) + b
    if score is not None:
        m += b"\x15" + struct.pack("<f", score)
    if tp is not None:
        m += b"\x18" + _vi(tp)
    m += extra
    return b"\x0a" + _vi(len(m)) + m


HAND = [("<unk>", 0.0, 2), ("<s>", 0.0, 3), ("</s>", 0.0, 3), ("<0x0A>", 0.0, 6), ("▁", -1.0, None), ("▁he", -2.0, 1), ("▁hell", -3.0, 1),
        ("llo", -4.0, 1), ("o", -5.0, 1), ("l", -6.0, 1), ("▁w", -7.0, 1), ("or", -8.0, 1), ("ld", -9.0, 1), ("é", -10.0, 1), ("h", -11.0, 1)]


def hand_model(with_newline=True):
    m = b""
    for i, (p, s, t) in enumerate(HAND):
        if p == "<0x0A>" and not with_newline:
            m += _piece(None, 0.5, 6)  # an entry without a string: skipped, but the ids of the later pieces still count it
        else:
            m += _piece(p, s, t, extra=b"\xc2\x0c\x01x" if i == 5 else b"")  # field 200 (an extension) is ignored
    m += b"\x12\x03\x08\x01\x10"  # field 2 (trainer_spec), skipped as a whole
    return m


def test_model_parsing_by_hand():
    t = Tokenizer.from_bytes(hand_model())
    assert len(t) == len(HAND)
    for i, (p, s, tp) in enumerate(HAND):
        kind, score, idx = t.piece_info(p)
        assert idx == i and score == np.float32(s) and t.str_to_id(p) == i and t.id_to_str(i) == p
        assert kind == {None: "Normal", 1: "Normal", 2: "Unknown", 3: "Control", 6: "Byte"}[tp]
    assert t.str_to_id("nope") is None
    with pytest.raises(IndexError):
        t.id_to_str(len(HAND))
    # without a string the entry is dropped but keeps its index; its id then has no piece (the reference panics)
    t2 = Tokenizer.from_bytes(hand_model(with_newline=False))
    assert len(t2) == len(HAND) - 1 and t2.str_to_id("▁") == 4 and t2.str_to_id("<0x0A>") is None
    with pytest.raises(IndexError):
        t2.id_to_str(3)
    # a repeated string keeps the later index; an unknown type is an error; truncated input is an error
    t3 = Tokenizer.from_bytes(_piece("a", 0.0, 1) + _piece("b", 0.0, 1) + _piece("a", 0.0, 1))
    assert t3.str_to_id("a") == 2 and t3.str_to_id("b") == 1 and len(t3) == 2
    with pytest.raises(TokenizerError, match="Unknown piece type"):
        Tokenizer.from_bytes(_piece("a", 0.0, 7))
    with pytest.raises(TokenizerError):
        Tokenizer.from_bytes(hand_model() + b"\x0a")
    with pytest.raises(TokenizerError):
        Tokenizer.from_bytes(b"\x0a\x05ab")


def test_matching_rules_by_hand():
    t = Tokenizer.from_bytes(hand_model())
    # longest piece that is a prefix wins at every position
    assert t.tokenize_to_pieces("▁hello") == ["▁hell", "o"]
    assert t.tokenize_to_pieces("▁helo") == ["▁he", "l", "o"]
    assert t.tokenize_to_pieces("▁world") == ["▁w", "or", "ld"]
    # tokenize_to_ids: "▁" in front, spaces become "▁", start token 1
    assert t.tokenize_to_ids("hello world") == [1, 6, 8, 10, 11, 12]
    assert t.tokenize_to_ids("") == [1, 4]
    assert t.tokenize_to_ids(" ") == [1, 4, 4]
    # a character without a piece is skipped byte by byte when the next byte starts a character ('x' is ASCII) ...
    assert t.tokenize_to_pieces("oxo") == ["o", "o"]
    # ... but skipping into the middle of a multi-byte character drops the rest of the text (str::get(1..) is None)
    assert t.tokenize_to_pieces("oüo") == ["o"]
    assert t.tokenize_to_pieces("oéo") == ["o", "é", "o"]
    # newline: the byte piece when the model has it, dropped otherwise
    assert t.tokenize_to_pieces("o\no") == ["o", "<0x0A>", "o"]
    assert t.tokenize_to_ids("h\nh") == [1, 4, 14, 3, 14]
    t2 = Tokenizer.from_bytes(hand_model(with_newline=False))
    assert t2.tokenize_to_pieces("o\no") == ["o", "o"]
    # control pieces are ordinary strings to this matcher
    assert t.tokenize_to_pieces("<s>o</s>") == ["<s>", "o", "</s>"]


@pytest.fixture(scope="module")
def trained_model(tmp_path_factory):
    spm = pytest.importorskip("sentencepiece")
    rng = np.random.default_rng(0)
    words = ["the", "quick", "brown", "fox", "jumps", "over", "lazy", "dog", "transformer", "attention", "token", "sampler", "wave", "front",
             "matrix", "core", "é", "naïve", "日本", "half", "float", "kernel", "cache", "rope", "norm"]
    corpus = [" ".join(rng.choice(words, size=rng.integers(3, 12))) for _ in range(400)]
    buf = io.BytesIO()
    spm.SentencePieceTrainer.train(sentence_iterator=iter(corpus), model_writer=buf, vocab_size=300, model_type="bpe", byte_fallback=True,
                                   character_coverage=1.0, bos_id=1, eos_id=2, unk_id=0, minloglevel=2)
    path = tmp_path_factory.mktemp("spm") / "tokenizer.model"
    path.write_bytes(buf.getvalue())
    return str(path), spm.SentencePieceProcessor(model_proto=buf.getvalue())


def test_model_parsing_against_sentencepiece(trained_model):
    path, sp = trained_model
    t = Tokenizer.load(path)
    assert len(t) == sp.get_piece_size()  # all strings distinct in a trained model
    for i in range(sp.get_piece_size()):
        piece = sp.id_to_piece(i)
        kind, score, idx = t.piece_info(piece)
        assert idx == i and t.id_to_str(i) == piece and score == np.float32(sp.get_score(i))
        want = "Unknown" if sp.is_unknown(i) else "Control" if sp.is_control(i) else "Byte" if sp.is_byte(i) else "Unused" if sp.is_unused(i) else "Normal"
        assert kind == want, (i, piece)
    assert t.str_to_id("<0x0A>") == sp.piece_to_id("<0x0A>")
    # every id the matcher produces names a piece that is a prefix of what was left (property of the matching rule)
    text = "the quick brown fox\njumps over the naïve 日本 dog"
    ids = t.tokenize_to_ids(text)
    assert ids[0] == 1
    rebuilt = "".join("\n" if t.id_to_str(i) == "<0x0A>" else t.id_to_str(i) for i in ids[1:])
    assert rebuilt == ("▁" + text).replace(" ", "▁")


def test_cpp_tokenizer_equals_python(trained_model, tmp_path):
    from rllama_amd import build
    exe = build.build_host()
    path, _ = trained_model
    hand = tmp_path / "hand.model"
    hand.write_bytes(hand_model())
    for model, texts in ((path, ["the quick brown fox", "naïve 日本\nkernel  cache", "", "zzz qqq", "é\n\né"]),
                         (str(hand), ["hello world", "oüo", "oxo", "h\nh", " "])):
        t = Tokenizer.load(model)
        for text in texts:
            r = subprocess.run([exe, "--tokenize", model, text], capture_output=True, text=True, timeout=60)
            assert r.returncode == 0, r.stderr
            ids = [int(v) for v in r.stdout.splitlines()[0].split()[1:]]
            assert ids == t.tokenize_to_ids(text), (model, text)
    r = subprocess.run([exe, "--tokenize", str(tmp_path / "missing.model"), "x"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 1 and "IO error" in r.stderr
