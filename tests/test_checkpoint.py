"""On-disk model format (Noeda/rllama src/unpickler.rs, src/data_source.rs, src/tensor.rs:2346-2546): the reader
against a hand-assembled pickle, against CPython's own pickle machinery and against files torch.save wrote; the
writer against the reader.  CPU only."""
import io
import json
import os
import pickle
import struct
import zipfile

import numpy as np
import pytest

from rllama_amd import checkpoint as ck


def _u(s):
    b = s.encode()
    return b"\x58" + struct.pack("<I", len(b)) + b


def _i(v):
    return b"\x4a" + struct.pack("<i", v)


def test_unpickle_hand_assembled_minimal_file():
    """Byte string put together by hand from the opcode table of src/unpickler.rs:317-675 (not by the writer)."""
    t2d = (_u("layers.0.attention.wq.weight") + b"ctorch._utils\n_rebuild_tensor_v2\n" + b"(" + b"(" + _u("storage") + b"ctorch\nHalfStorage\n"
           + _u("7") + _u("cpu") + _i(12) + b"t" + b"Q" + _i(0) + _i(3) + _i(4) + b"\x86" + _i(4) + _i(1) + b"\x86" + b"\x89"
           + b"ccollections\nOrderedDict\n" + b")" + b"R" + b"t" + b"R")
    t1d = (_u("norm.weight") + b"ctorch._utils\n_rebuild_tensor_v2\n" + b"(" + b"(" + _u("storage") + b"ctorch\nHalfStorage\n"
           + _u("8") + _u("cpu") + _i(4) + b"t" + b"Q" + _i(0) + _i(4) + b"\x85" + _i(1) + b"\x85" + b"\x89"
           + b"ccollections\nOrderedDict\n" + b")" + b"R" + b"t" + b"R")
    data = b"\x80\x02" + b"}" + b"(" + t2d + t1d + b"u" + b"."
    v = ck.unpickle(data)
    assert set(v) == {"layers.0.attention.wq.weight", "norm.weight"}
    wq = v["layers.0.attention.wq.weight"]
    assert wq.callable == ck.Global("torch._utils", "_rebuild_tensor_v2")
    assert wq.args[0] == ck.PersistentId(("storage", ck.Global("torch", "HalfStorage"), "7", "cpu", 12))
    assert wq.args[1:5] == (0, (3, 4), (4, 1), False)
    assert wq.args[5] == ck.Reduce(ck.Global("collections", "OrderedDict"), ())
    b = ck.to_tensor_builder(wq, "layers.0.attention.wq.weight")
    assert (b.src_path, b.rows, b.cols, b.stride, b.nitems, b.offset) == ("7", 3, 4, 4, 12, 0)
    b1 = ck.to_tensor_builder(v["norm.weight"], "norm.weight")
    assert (b1.rows, b1.cols, b1.stride) == (1, 4, 1)  # 1-D tensors load as 1 x n (src/unpickler.rs:207-212)


def test_unpickle_opcode_details():
    # BININT2 is read as a signed 16-bit value (src/unpickler.rs:484); BININT1 unsigned; memo put / get both widths
    assert ck.unpickle(b"\x80\x02M\xff\xff.") == -1
    assert ck.unpickle(b"\x80\x02M\x00\x80.") == -32768
    assert ck.unpickle(b"\x80\x02K\xff.") == 255
    assert ck.unpickle(b"\x80\x02J\xfe\xff\xff\xff.") == -2
    assert ck.unpickle(b"\x80\x02(K\x01q\x05h\x05r\x00\x01\x00\x00j\x00\x01\x00\x00t.") == (1, 1, 1)
    assert ck.unpickle(b"\x80\x02}(K\x01K\x02K\x03K\x04u(K\x05K\x06u.") == {1: 2, 3: 4, 5: 6}
    assert ck.unpickle(b"\x80\x02K\x01\x85.") == (1,) and ck.unpickle(b"\x80\x02).") == ()
    # trailing bytes after STOP are ignored; without STOP the stack must still hold exactly one value
    assert ck.unpickle(b"\x80\x02K\x07.garbage") == 7
    assert ck.unpickle(b"\x80\x02K\x07") == 7


REJECTED_PICKLES = [
    (b"", "too short"), (b"\x80\x03K\x01.", "magic"), (b"\x80\x02\x8a\x01\x01.", "Unknown opcode: 138"), (b"\x80\x02K\x01K\x02\x87.", "Unknown opcode: 135"),
    (b"\x80\x02K\x01K\x02.", "exactly one"), (b"\x80\x02K\x01t.", "No mark"), (b"\x80\x02h\x00.", "BINGET index"), (b"\x80\x02X\x05\x00\x00\x00ab", "BINUNICODE"),
    (b"\x80\x02K\x01(K\x02K\x03u.", "SETITEMS on non-dict"), (b"\x80\x02}(K\x01u.", "Unexpected mark"), (b"\x80\x02J\x01\x02", "BININT"),
    (b"\x80\x02N.", "Unknown opcode: 78"),
]


@pytest.mark.parametrize("data,msg", REJECTED_PICKLES)
def test_unpickle_rejects(data, msg):
    with pytest.raises(ck.UnpicklingError, match=msg):
        ck.unpickle(data)


class _PyLoader(pickle.Unpickler):
    """CPython's unpickler with classes and persistent ids mapped onto the reader's value types: an independent
    implementation of the pickle grammar to compare the reader with."""

    def find_class(self, module, name):
        g = ck.Global(module, name)

        class _Call:
            def __call__(self, *args):
                return ck.Reduce(g, tuple(args))

            def __eq__(self, other):
                return other == g

            def __hash__(self):
                return hash(g)
        c = _Call()
        c.g = g
        return c

    def persistent_load(self, pid):
        return ck.PersistentId(pid)


def _normalise(v):
    if hasattr(v, "g"):
        return v.g
    if isinstance(v, ck.Reduce):
        return ck.Reduce(_normalise(v.callable), _normalise(v.args))
    if isinstance(v, ck.PersistentId):
        return ck.PersistentId(_normalise(v.value))
    if isinstance(v, tuple):
        return tuple(_normalise(x) for x in v)
    if isinstance(v, dict):
        return {k: _normalise(x) for k, x in v.items()}
    return v


def test_writer_output_reads_the_same_through_cpython_pickle():
    entries = [("tok_embeddings.weight", "0", (96, 64)), ("norm.weight", "1", (64,)), ("layers.0.feed_forward.w2.weight", "2", (64, 192)),
               ("layers.11.attention_norm.weight", "3", (64,)), ("output.weight", "4", (70000, 4))]
    data = ck.pickle_state_dict(entries)
    mine = ck.unpickle(data)
    theirs = _normalise(_PyLoader(io.BytesIO(data)).load())
    assert mine == theirs
    for name, key, shape in entries:
        b = ck.to_tensor_builder(mine[name], name)
        assert b.src_path == key and b.nitems == int(np.prod(shape)) and b.offset == 0
        assert (b.rows, b.cols) == (shape if len(shape) == 2 else (1, shape[0]))


def test_reader_on_a_file_torch_wrote(tmp_path):
    """torch.save of a half-precision state dict, unzipped the way the reference's README asks for, is read back
    exactly: the reader agrees with the program that defines the format."""
    torch = pytest.importorskip("torch")
    g = torch.Generator().manual_seed(5)
    sd = {"tok_embeddings.weight": torch.randn(40, 16, generator=g).half(), "norm.weight": torch.rand(16, generator=g).half(),
          "output.weight": torch.randn(40, 16, generator=g).half()}
    for l in range(2):
        for nm, shp in (("attention.wq", (16, 16)), ("attention.wk", (16, 16)), ("attention.wv", (16, 16)), ("attention.wo", (16, 16)),
                        ("feed_forward.w1", (48, 16)), ("feed_forward.w2", (16, 48)), ("feed_forward.w3", (48, 16))):
            sd[f"layers.{l}.{nm}.weight"] = torch.randn(*shp, generator=g).half()
        sd[f"layers.{l}.attention_norm.weight"] = torch.rand(16, generator=g).half()
        sd[f"layers.{l}.ffn_norm.weight"] = torch.rand(16, generator=g).half()
    model = tmp_path / "m"
    (model / "consolidated.00").mkdir(parents=True)
    torch.save(sd, str(tmp_path / "consolidated.00.pth"))
    with zipfile.ZipFile(tmp_path / "consolidated.00.pth") as z:
        for info in z.infolist():
            rel = info.filename.split("/", 1)[1]  # drop the archive's top directory
            if rel == "data.pkl" or rel.startswith("data/"):
                dst = model / "consolidated.00" / rel
                dst.parent.mkdir(parents=True, exist_ok=True)
                dst.write_bytes(z.read(info))
    (model / "params.json").write_text(json.dumps({"dim": 16, "multiple_of": 8, "n_heads": 2, "n_layers": 2, "norm_eps": 1e-6, "vocab_size": -1}))
    c = ck.Checkpoint(str(model))
    assert (c.dim, c.n_heads, c.n_layers, c.norm_eps, c.vocab_size) == (16, 2, 2, 1e-6, -1)
    assert set(c.tensor_names()) == set(sd)
    for name, t in sd.items():
        got = c.load_f16_bits(name, ck.FROM_PIECES_ROWS)
        want = t.numpy().view(np.uint16).reshape(got.shape)
        assert np.array_equal(got, want), name


def test_write_then_read_one_and_two_shards(tmp_path):
    rng = np.random.default_rng(3)
    d, F, V, L = 32, 96, 50, 2
    T = {"tok_embeddings.weight": rng.integers(0, 65536, (V, d), dtype=np.uint16), "norm.weight": rng.integers(0, 65536, d, dtype=np.uint16),
         "output.weight": rng.integers(0, 65536, (V, d), dtype=np.uint16)}
    for l in range(L):
        for nm, shp in (("attention.wq", (d, d)), ("attention.wk", (d, d)), ("attention.wv", (d, d)), ("attention.wo", (d, d)),
                        ("feed_forward.w1", (F, d)), ("feed_forward.w2", (d, F)), ("feed_forward.w3", (F, d))):
            T[f"layers.{l}.{nm}.weight"] = rng.integers(0, 65536, shp, dtype=np.uint16)
        T[f"layers.{l}.attention_norm.weight"] = rng.integers(0, 65536, d, dtype=np.uint16)
        T[f"layers.{l}.ffn_norm.weight"] = rng.integers(0, 65536, d, dtype=np.uint16)
    params = {"dim": d, "n_heads": 4, "n_layers": L, "norm_eps": 1e-5, "vocab_size": V}
    for shards in (1, 2):
        path = str(tmp_path / f"s{shards}")
        ck.write_checkpoint(path, params, T, n_shards=shards)
        assert sorted(os.listdir(path)) == ["consolidated.%02d" % i for i in range(shards)] + ["params.json"]
        c = ck.Checkpoint(path)
        assert len(c.shards) == shards and c.norm_eps == 1e-5
        for key, (name, direction, first) in ck._TOP.items():
            assert np.array_equal(c.load_f16_bits(name, direction, first), T[name].reshape(-1, T[name].shape[-1]))
        for l in range(L):
            for key, (fmt, direction, first) in ck._LAYER.items():
                name = fmt.format(l)
                assert np.array_equal(c.load_f16_bits(name, direction, first), T[name].reshape(-1, T[name].shape[-1])), (shards, name)
    # joined the wrong way round, a split matrix comes out different: the direction matters
    c = ck.Checkpoint(str(tmp_path / "s2"))
    assert c.load_f16_bits("layers.0.attention.wo.weight", ck.FROM_PIECES_ROWS).shape == (2 * d, d // 2)


def test_checkpoint_errors(tmp_path):
    with pytest.raises(FileNotFoundError):
        ck.Checkpoint(str(tmp_path))  # no params.json: unknown source
    (tmp_path / "params.json").write_text(json.dumps({"hidden_size": 8, "num_attention_heads": 2, "num_hidden_layers": 1, "rms_norm_eps": 1e-6, "vocab_size": 9}))
    c = ck.Checkpoint(str(tmp_path))  # the aliases of src/model_params.rs are accepted; no shards yet
    assert (c.dim, c.n_heads, c.n_layers, c.vocab_size) == (8, 2, 1, 9) and c.shards == []
    with pytest.raises(KeyError):
        c.load_f16_bits("norm.weight", ck.FROM_PIECES_ROWS, True)
    # float storage, a transposed (non-contiguous) view and a 3-D tensor are not tensors the reference loads
    ok = ck.unpickle(ck.pickle_state_dict([("a", "0", (2, 3))]))["a"]
    assert ck.to_tensor_builder(ok, "a") is not None
    args = ok.args
    bad_storage = ck.Reduce(ok.callable, (ck.PersistentId(("storage", ck.Global("torch", "FloatStorage"), "0", "cpu", 6)),) + args[1:])
    bad_stride = ck.Reduce(ok.callable, args[:3] + ((1, 2),) + args[4:])
    bad_rank = ck.Reduce(ok.callable, args[:2] + ((1, 2, 3), (6, 3, 1)) + args[4:])
    for bad in (bad_storage, bad_stride, bad_rank, ck.Reduce(ck.Global("torch._utils", "_rebuild_tensor"), args), "x"):
        assert ck.to_tensor_builder(bad, "a") is None


def _fnv1a(bits: np.ndarray) -> int:
    h = 1469598103934665603
    for b in np.ascontiguousarray(bits).astype("<u2").tobytes():
        h = ((h ^ b) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return h


def test_cpp_host_loader_reads_what_the_python_writer_wrote(tmp_path):
    """The C++ mirror of the reader (rllama_amd/host/model_files.hpp), through the host example's --inspect mode:
    same parameters, same shapes, same bits (two shards, joined by rows or columns as the reference does)."""
    import subprocess
    from rllama_amd import build
    exe = build.build_host()
    rng = np.random.default_rng(9)
    d, F, V, L = 16, 48, 20, 2
    T = {"tok_embeddings.weight": rng.integers(0, 65536, (V, d), dtype=np.uint16), "norm.weight": rng.integers(0, 65536, d, dtype=np.uint16),
         "output.weight": rng.integers(0, 65536, (V, d), dtype=np.uint16)}
    for l in range(L):
        for nm, shp in (("attention.wq", (d, d)), ("attention.wk", (d, d)), ("attention.wv", (d, d)), ("attention.wo", (d, d)),
                        ("feed_forward.w1", (F, d)), ("feed_forward.w2", (d, F)), ("feed_forward.w3", (F, d))):
            T[f"layers.{l}.{nm}.weight"] = rng.integers(0, 65536, shp, dtype=np.uint16)
        T[f"layers.{l}.attention_norm.weight"] = rng.integers(0, 65536, d, dtype=np.uint16)
        T[f"layers.{l}.ffn_norm.weight"] = rng.integers(0, 65536, d, dtype=np.uint16)
    path = str(tmp_path / "m2")
    ck.write_checkpoint(path, {"dim": d, "n_heads": 2, "n_layers": L, "norm_eps": 1e-6, "vocab_size": V, "note": {"nested": [1, "}"]}}, T, n_shards=2)
    r = subprocess.run([exe, "--inspect", path], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stderr
    lines = r.stdout.strip().splitlines()
    assert lines[0] == f"params dim={d} n_heads=2 n_layers={L} norm_eps=1e-06 vocab_size={V} shards=2"
    seen = {}
    for ln in lines[1:]:
        _, name, rows, cols, h = ln.split()
        seen[name] = (int(rows), int(cols), int(h, 16))
    assert set(seen) == set(T)
    for name, arr in T.items():
        a2 = arr.reshape(-1, arr.shape[-1])
        assert seen[name] == (a2.shape[0], a2.shape[1], _fnv1a(a2)), name
    # and the failure path: a directory without params.json
    r = subprocess.run([exe, "--inspect", str(tmp_path)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 1 and "Unknown source" in r.stderr


def test_synthetic_checkpoint_matches_the_generator(tmp_path):
    """The benchmark model written to disk holds exactly the generator's bits (the weights every other test uses)."""
    import rllama_amd
    path = str(tmp_path / "syn")
    ck.write_synthetic_checkpoint(path, dim=64, n_layers=2, n_heads=2, ffn_hidden=192, vocab_size=96, seed=3, n_shards=2)
    c = ck.Checkpoint(path)
    assert (c.dim, c.n_layers, c.n_heads, c.vocab_size, c.norm_eps) == (64, 2, 2, 96, 1e-6)
    w2 = c.load_f16_bits("layers.1.feed_forward.w2.weight", ck.FROM_PIECES_COLS)
    assert np.array_equal(w2, rllama_amd.synth_normal_f16(3, rllama_amd.W2, 1, 64 * 192).reshape(64, 192))
    emb = c.load_f16_bits("tok_embeddings.weight", ck.FROM_PIECES_COLS)
    assert np.array_equal(emb, rllama_amd.synth_normal_f16(3, rllama_amd.TOK_EMB, 0, 96 * 64).reshape(96, 64))
    assert np.all(c.load_f16_bits("layers.0.ffn_norm.weight", ck.FROM_PIECES_ROWS, True) == 0x3C00)


def _hostile_dir(tmp_path, tag, entries_by_shard, files):
    """A model directory whose data.pkl files hold `entries_by_shard[i]` and whose data/ folders hold `files[i]`."""
    path = tmp_path / tag
    path.mkdir()
    (path / "params.json").write_text(json.dumps({"dim": 8, "n_heads": 2, "n_layers": 1, "norm_eps": 1e-6, "vocab_size": 4}))
    for i, entries in enumerate(entries_by_shard):
        sd = path / f"consolidated.{i:02d}"
        (sd / "data").mkdir(parents=True)
        (sd / "data.pkl").write_bytes(ck.pickle_state_dict(entries))
        for key, n in files[i].items():
            (sd / "data" / key).write_bytes(np.arange(n, dtype="<u2").tobytes())
    return str(path)


DAMAGED_CHECKPOINTS = [
    # negative extents (BININT is signed, src/unpickler.rs:414): one shard claims 6 columns, the other -4, so the sum (2) would
    # size the joined matrix while the first shard still copies 6 columns per row
    ("mixed_sign_cols", [[("w", "0", (3, 6))], [("w", "0", (3, -4))]], "invalid stride|does not fit its storage"),
    ("negative_rows", [[("w", "0", (-2, 4))]], "does not fit its storage"),
    ("zero_cols", [[("w", "0", (0,))]], "does not fit its storage"),
    ("negative_cols_1d", [[("w", "0", (-4,), 0, 8)]], "does not fit its storage"),
    ("negative_offset", [[("w", "0", (2, 4), -1, 8)]], "does not fit its storage"),
    ("past_the_storage", [[("w", "0", (2, 4), 4, 8)]], "does not fit its storage"),
    # the storage key must stay a file name inside consolidated.NN/data/
    ("dotdot_key", [[("w", "../../params.json", (1, 2))]], "not a plain file name"),
    ("absolute_key", [[("w", "/etc/hostname", (1, 2))]], "not a plain file name"),
]


@pytest.mark.parametrize("tag,entries,msg", DAMAGED_CHECKPOINTS)
def test_damaged_checkpoints_fail_cleanly_in_both_readers(tmp_path, tag, entries, msg):
    """Extents and storage keys come from the pickle unchecked; both readers must refuse them before sizing a buffer or
    opening a path (the reference panics on the same inputs: usize casts of negative i64 and slice bounds)."""
    import subprocess
    from rllama_amd import build
    files = [{"0": 64} for _ in entries]
    path = _hostile_dir(tmp_path, tag, entries, files)
    with pytest.raises(ValueError, match=msg):
        ck.Checkpoint(path).load_f16_bits("w", ck.FROM_PIECES_COLS)
    r = subprocess.run([build.build_host(), "--inspect", path], capture_output=True, text=True, timeout=60)
    import re
    assert r.returncode == 1 and re.search(msg, r.stderr), (r.returncode, r.stderr)


def test_offset_and_item_count_are_honoured(tmp_path):
    """A piece that starts inside its storage file reads from there (storage offset in elements, src/tensor.rs:2452-2480)."""
    path = _hostile_dir(tmp_path, "off", [[("w", "0", (2, 3), 5, 16)]], [{"0": 16}])
    got = ck.Checkpoint(path).load_f16_bits("w", ck.FROM_PIECES_ROWS)
    assert np.array_equal(got, np.arange(5, 11, dtype=np.uint16).reshape(2, 3))
