"""The CPU-only pieces that parse untrusted bytes or index by computed extents -- the C++ file readers of the host layer
(rllama_amd/host/model_files.hpp: the pickle subset of src/unpickler.rs:317-675, params.json, shard joining of
src/data_source.rs:166-210; tokenizer.hpp) and the CPU oracle -- built with AddressSanitizer + UndefinedBehaviorSanitizer
(`python -m rllama_amd.build --host-asan`, `make -C oracle asan`) and run over the suite's good, damaged and mutated
inputs.  A reader may refuse an input (exit code 1 with a message); it may never trip a sanitizer.  CPU only: nothing of the
device library is built this way."""
import json
import os
import re
import subprocess

import numpy as np
import pytest

from rllama_amd import build
from rllama_amd import checkpoint as ck
from test_checkpoint import DAMAGED_CHECKPOINTS, REJECTED_PICKLES, _hostile_dir
from test_tokenizer import hand_model

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SAN_ENV = dict(os.environ, ASAN_OPTIONS="exitcode=99:abort_on_error=0:detect_leaks=1", UBSAN_OPTIONS="halt_on_error=1:exitcode=98:print_stacktrace=1")


@pytest.fixture(scope="module")
def checker():
    return build.build_host_asan()


def run(checker, *args):
    r = subprocess.run([checker, *args], capture_output=True, text=True, errors="replace", timeout=120, env=SAN_ENV)
    assert r.returncode in (0, 1), f"{args}: exit code {r.returncode}\n{r.stderr[-3000:]}"
    assert "Sanitizer" not in r.stderr and "runtime error" not in r.stderr, r.stderr[-3000:]
    return r


def test_oracle_under_the_sanitizers():
    subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "asan"], stdout=subprocess.DEVNULL)
    r = subprocess.run([os.path.join(ROOT, "oracle", "_build", "oracle_asan_check")], capture_output=True, text=True, timeout=600, env=SAN_ENV)
    assert r.returncode == 0, f"exit code {r.returncode}\n{r.stdout[-500:]}\n{r.stderr[-3000:]}"
    assert "every entry point ran" in r.stdout


def test_good_checkpoint_reads_the_same_under_the_sanitizers(checker, tmp_path):
    path = str(tmp_path / "syn")
    ck.write_synthetic_checkpoint(path, dim=64, n_layers=2, n_heads=2, ffn_hidden=192, vocab_size=96, seed=3, n_shards=2)
    r = run(checker, "inspect", path)
    assert r.returncode == 0, r.stderr
    plain = subprocess.run([build.build_host(), "--inspect", path], capture_output=True, text=True, timeout=120)
    assert plain.returncode == 0 and r.stdout == plain.stdout and r.stdout.count("\ntensor ") == 21


@pytest.mark.parametrize("tag,entries,msg", DAMAGED_CHECKPOINTS)
def test_damaged_checkpoints_under_the_sanitizers(checker, tmp_path, tag, entries, msg):
    path = _hostile_dir(tmp_path, tag, entries, [{"0": 64} for _ in entries])
    r = run(checker, "inspect", path)
    assert r.returncode == 1 and re.search(msg, r.stderr), r.stderr


def test_rejected_and_mutated_pickles_under_the_sanitizers(checker, tmp_path):
    """The reader's own error cases, every prefix of a valid data.pkl, and 400 variants of it with bytes overwritten,
    inserted or dropped (extents, opcodes, string lengths and memo indices all get hit)."""
    for i, (data, msg) in enumerate(REJECTED_PICKLES):
        f = tmp_path / f"rej{i}.pkl"
        f.write_bytes(data)
        r = run(checker, "unpickle", str(f))
        assert r.returncode == 1 and re.search(msg, r.stderr), (data, r.stderr)
    good = ck.pickle_state_dict([("layers.0.attention.wq.weight", "0", (4, 6)), ("norm.weight", "1", (6,)), ("tok_embeddings.weight", "2", (5, 6), 3, 40)])
    f = tmp_path / "good.pkl"
    f.write_bytes(good)
    assert run(checker, "unpickle", str(f)).returncode == 0
    f = tmp_path / "v.pkl"
    refused = 0
    for n in range(len(good)):
        f.write_bytes(good[:n])
        refused += run(checker, "unpickle", str(f)).returncode
    # (a prefix that leaves exactly one value on the stack is a pickle to the reference too, src/unpickler.rs:656-675: the
    # empty dict after three bytes, and the whole dict without its STOP)
    assert refused >= len(good) - 3
    rng = np.random.default_rng(7)
    outcomes = {0: 0, 1: 0}
    for _ in range(400):
        b = bytearray(good)
        for _ in range(int(rng.integers(1, 4))):
            pos = int(rng.integers(2, len(b)))
            kind = int(rng.integers(0, 3))
            if kind == 0:
                b[pos] = int(rng.integers(0, 256))
            elif kind == 1:
                b.insert(pos, int(rng.integers(0, 256)))
            else:
                del b[pos]
        f.write_bytes(bytes(b))
        outcomes[run(checker, "unpickle", str(f)).returncode] += 1
    assert outcomes[1] > 100, outcomes                # most damage is noticed; none of it may trip a sanitizer


def test_mutated_checkpoint_directories_under_the_sanitizers(checker, tmp_path):
    """The whole path from data.pkl to joined tensors on mutated pickles whose data files are short: extents that survive the
    pickle reader meet the file sizes."""
    entries = [("w", "0", (3, 4)), ("layers.0.feed_forward.w2.weight", "1", (2, 8), 2, 20)]
    good = ck.pickle_state_dict(entries)
    rng = np.random.default_rng(11)
    for i in range(120):
        d = tmp_path / f"m{i}"
        (d / "consolidated.00" / "data").mkdir(parents=True)
        (d / "params.json").write_text(json.dumps({"dim": 8, "n_heads": 2, "n_layers": 1, "norm_eps": 1e-6, "vocab_size": 4}) if i % 7 else '{"dim": [1, {"a": "}"}], "n_heads"')
        b = bytearray(good)
        for _ in range(int(rng.integers(0, 3))):
            b[int(rng.integers(2, len(b)))] = int(rng.integers(0, 256))
        (d / "consolidated.00" / "data.pkl").write_bytes(bytes(b))
        (d / "consolidated.00" / "data" / "0").write_bytes(np.arange(12 if i % 3 else 5, dtype="<u2").tobytes())
        (d / "consolidated.00" / "data" / "1").write_bytes(np.arange(20 if i % 2 else 7, dtype="<u2").tobytes())
        run(checker, "inspect", str(d))


def test_tokenizer_model_files_under_the_sanitizers(checker, tmp_path):
    good = hand_model()
    f = tmp_path / "tok.model"
    f.write_bytes(good)
    r = run(checker, "tokenize", str(f), "hello world\nhé")
    assert r.returncode == 0 and r.stdout.startswith("ids: 1 ")
    plain = subprocess.run([build.build_host(), "--tokenize", str(f), "hello world\nhé"], capture_output=True, text=True, timeout=60)
    assert plain.stdout == r.stdout
    for n in range(0, len(good), 3):                  # truncated files: a length prefix that points past the end, a cut varint
        f.write_bytes(good[:n])
        run(checker, "tokenize", str(f), "hello")
    rng = np.random.default_rng(5)
    for _ in range(200):
        b = bytearray(good)
        for _ in range(int(rng.integers(1, 4))):
            b[int(rng.integers(0, len(b)))] = int(rng.integers(0, 256))
        f.write_bytes(bytes(b))
        run(checker, "tokenize", str(f), "hello wor\xe9ld ▁x")
