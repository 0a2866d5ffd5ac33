"""The reference's on-disk model format (the original LLaMA release, unzipped): reader, writer, loader.

Layout (Noeda/rllama src/data_source.rs:166-210):

    <model>/params.json                      dim, n_heads, n_layers, norm_eps, vocab_size (src/model_params.rs:3-14)
    <model>/consolidated.NN/data.pkl         pickle protocol 2, a dict  name -> torch._utils._rebuild_tensor_v2(...)
    <model>/consolidated.NN/data/<key>       raw little-endian f16, row-major, no header

NN counts shards from 00; a tensor split over shards is put together by rows (wq wk wv w1 w3 output) or by
columns (wo w2 tok_embeddings), norm weights are taken from shard 0 (src/transformer.rs:297-304, 405-412, 456-467,
490-503, 595-614; src/embedding.rs:18-37; src/tensor.rs:2335-2343).

`unpickle` accepts exactly the opcode subset of src/unpickler.rs:317-675 and builds the same value tree; in
particular BININT2 is read as a *signed* 16-bit integer like :484 does.  It executes nothing from the file.
"""
from __future__ import annotations

import json
import os
import struct
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

# ---------------------------------------------------------------------------------------------------------------
# value tree (src/unpickler.rs:23-34)


@dataclass(frozen=True)
class Global:
    module: str
    name: str


@dataclass(frozen=True)
class PersistentId:
    value: object


@dataclass(frozen=True)
class Reduce:
    callable: object
    args: object


class _Mark:
    pass


class UnpicklingError(Exception):
    pass


def unpickle(data: bytes):
    """src/unpickler.rs:317-675.  Returns str / int / bool / tuple / dict / Global / PersistentId / Reduce."""
    if len(data) < 2:
        raise UnpicklingError("Data is too short to be a pickle")
    if data[0] != 0x80 or data[1] != 2:
        raise UnpicklingError("No magic header using Pickle 2 protocol")
    memo: Dict[int, object] = {}
    stack: List[object] = []
    pos = 2
    n = len(data)

    def need(k: int, what: str):
        if pos + k > n:
            raise UnpicklingError(f"Unexpected end of data while handling {what}")

    def pop_to_mark(what: str) -> List[object]:
        items: List[object] = []
        while stack:
            top = stack.pop()
            if isinstance(top, _Mark):
                items.reverse()
                return items
            items.append(top)
        raise UnpicklingError(f"No mark while handling {what}")

    while pos < n:
        op = data[pos]
        if op == 0x7D:  # EMPTY_DICT
            stack.append({})
            pos += 1
        elif op == 0x71:  # BINPUT
            need(2, "BINPUT")
            if not stack:
                raise UnpicklingError("Stack is empty while handling BINPUT")
            memo[data[pos + 1]] = stack[-1]
            pos += 2
        elif op == 0x72:  # LONG_BINPUT
            need(5, "LONG_BINPUT")
            if not stack:
                raise UnpicklingError("Stack is empty while handling LONG_BINPUT")
            memo[struct.unpack_from("<I", data, pos + 1)[0]] = stack[-1]
            pos += 5
        elif op == 0x68:  # BINGET
            need(2, "BINGET")
            if data[pos + 1] not in memo:
                raise UnpicklingError("BINGET index out of range")
            stack.append(memo[data[pos + 1]])
            pos += 2
        elif op == 0x6A:  # LONG_BINGET
            need(5, "LONG_BINGET")
            key = struct.unpack_from("<I", data, pos + 1)[0]
            if key not in memo:
                raise UnpicklingError("LONG_BINGET index out of range")
            stack.append(memo[key])
            pos += 5
        elif op == 0x28:  # MARK
            stack.append(_Mark())
            pos += 1
        elif op == 0x58:  # BINUNICODE
            need(5, "BINUNICODE")
            ln = struct.unpack_from("<I", data, pos + 1)[0]
            need(5 + ln, "BINUNICODE")
            try:
                stack.append(data[pos + 5:pos + 5 + ln].decode("utf-8"))
            except UnicodeDecodeError as e:
                raise UnpicklingError("UTF-8 decoding error") from e
            pos += 5 + ln
        elif op == 0x63:  # GLOBAL: two newline-terminated names
            e1 = data.find(b"\n", pos + 1)
            e2 = data.find(b"\n", e1 + 1) if e1 >= 0 else -1
            if e1 < 0 or e2 < 0:
                raise UnpicklingError("Unexpected end of data while handling GLOBAL")
            stack.append(Global(data[pos + 1:e1].decode("latin-1"), data[e1 + 1:e2].decode("latin-1")))
            pos = e2 + 1
        elif op == 0x4A:  # BININT, signed 32 bit
            need(5, "BININT")
            stack.append(struct.unpack_from("<i", data, pos + 1)[0])
            pos += 5
        elif op == 0x4B:  # BININT1
            need(2, "BININT1")
            stack.append(data[pos + 1])
            pos += 2
        elif op == 0x4D:  # BININT2, read as SIGNED 16 bit (src/unpickler.rs:484)
            need(3, "BININT2")
            stack.append(struct.unpack_from("<h", data, pos + 1)[0])
            pos += 3
        elif op == 0x74:  # TUPLE
            if not stack:
                raise UnpicklingError("Stack is empty while handling TUPLE")
            stack.append(tuple(pop_to_mark("TUPLE")))
            pos += 1
        elif op == 0x85:  # TUPLE1
            if not stack:
                raise UnpicklingError("Stack is empty while handling TUPLE1")
            stack.append((stack.pop(),))
            pos += 1
        elif op == 0x86:  # TUPLE2
            if len(stack) < 2:
                raise UnpicklingError("Stack does not have enough items while handling TUPLE2")
            b, a = stack.pop(), stack.pop()
            stack.append((a, b))
            pos += 1
        elif op == 0x29:  # EMPTY_TUPLE
            stack.append(())
            pos += 1
        elif op == 0x89:  # NEWFALSE
            stack.append(False)
            pos += 1
        elif op == 0x51:  # BINPERSID
            if not stack:
                raise UnpicklingError("Stack is empty while handling BINPERSID")
            stack.append(PersistentId(stack.pop()))
            pos += 1
        elif op == 0x52:  # REDUCE
            if len(stack) < 2:
                raise UnpicklingError("Stack does not have enough items while handling REDUCE")
            args, fn = stack.pop(), stack.pop()
            stack.append(Reduce(fn, args))
            pos += 1
        elif op == 0x75:  # SETITEMS
            if not stack:
                raise UnpicklingError("Stack is empty while handling SETITEMS")
            items = pop_to_mark("SETITEMS")
            if len(items) % 2:
                raise UnpicklingError("Unexpected mark while handling SETITEMS")
            if not stack:
                raise UnpicklingError("Stack is empty while handling SETITEMS")
            if not isinstance(stack[-1], dict):
                raise UnpicklingError("SETITEMS on non-dict")
            for i in range(0, len(items), 2):
                stack[-1][items[i]] = items[i + 1]
            pos += 1
        elif op == 0x2E:  # STOP
            break
        else:
            raise UnpicklingError(f"Unknown opcode: {op}")
    if len(stack) != 1:
        raise UnpicklingError("Stack does not have exactly one item after unpickling")
    return stack[0]


# ---------------------------------------------------------------------------------------------------------------
# tensor records (TensorBuilder, src/unpickler.rs:147-264 and src/tensor.rs:2346-2546)


@dataclass
class TensorBuilder:
    src_path: str
    tensor_name: str
    rows: int
    cols: int
    stride: int
    nitems: int
    offset: int


def to_tensor_builder(value, tensor_name: str) -> Optional[TensorBuilder]:
    """None for anything that is not a contiguous 1-D / 2-D HalfStorage tensor (src/unpickler.rs:147-249)."""
    if not (isinstance(value, Reduce) and value.callable == Global("torch._utils", "_rebuild_tensor_v2")):
        return None
    args = value.args
    if not (isinstance(args, tuple) and len(args) == 6 and isinstance(args[0], PersistentId)):
        return None
    st = args[0].value
    if not (isinstance(st, tuple) and len(st) >= 5 and st[0] == "storage" and st[1] == Global("torch", "HalfStorage")):
        return None
    if not (isinstance(st[2], str) and type(st[4]) is int and type(args[1]) is int):
        return None
    shape, stride = args[2], args[3]
    if not (isinstance(shape, tuple) and isinstance(stride, tuple) and len(shape) in (1, 2) and len(stride) in (1, 2)):
        return None
    if not all(type(v) is int for v in shape + stride):
        return None
    rows, cols = (shape[0], shape[1]) if len(shape) == 2 else (1, shape[0])
    if len(stride) == 1:
        if stride[0] != 1:
            return None
        row_stride = 1
    else:
        row_stride, col_stride = stride
        if col_stride != 1 or row_stride != cols:
            return None
    return TensorBuilder(st[2], tensor_name, rows, cols, row_stride, st[4], args[1])


FROM_PIECES_ROWS, FROM_PIECES_COLS = "rows", "cols"  # FromPiecesDirection (src/tensor.rs:2339-2343)


class Checkpoint:
    """DataSource::LLaMASource (src/data_source.rs:27-31, 166-197): the parsed data.pkl of every shard."""

    def __init__(self, path: str):
        self.path = path
        params_path = os.path.join(path, "params.json")
        if not os.path.exists(params_path):  # from_inferred_source (src/data_source.rs:198-210)
            raise FileNotFoundError(f"{params_path}: not a LLaMA-format model directory (Unknown source)")
        with open(params_path, "r") as f:
            p = json.load(f)

        def key(a, b=None):
            if a in p:
                return p[a]
            if b is not None and b in p:
                return p[b]
            raise KeyError(f"params.json: missing field {a}")

        # aliases of src/model_params.rs:5-12
        self.dim = int(key("dim", "hidden_size"))
        self.n_heads = int(key("n_heads", "num_attention_heads"))
        self.n_layers = int(key("n_layers", "num_hidden_layers"))
        self.norm_eps = float(key("norm_eps", "rms_norm_eps"))
        self.vocab_size = int(key("vocab_size"))
        self.shards: List[dict] = []
        part = 0
        while True:
            pkl = os.path.join(path, f"consolidated.{part:02d}", "data.pkl")
            if not os.path.exists(pkl):
                break
            with open(pkl, "rb") as f:
                v = unpickle(f.read())
            if not isinstance(v, dict):
                raise UnpicklingError(f"{pkl}: top-level value is not a dict")
            self.shards.append(v)
            part += 1

    def tensor_names(self) -> List[str]:
        return sorted(k for k in (self.shards[0] if self.shards else {}) if isinstance(k, str))

    def _builders(self, name: str, first_only: bool) -> List[TensorBuilder]:
        out = []
        for sh in self.shards:
            if name not in sh:
                raise KeyError(f"Missing field {name}")
            b = to_tensor_builder(sh[name], name)
            if b is None:
                raise UnpicklingError(f"{name}: data has incorrect format to be converted to a tensor")
            out.append(b)
            if first_only:
                break
        if not out:
            raise KeyError(f"Missing field {name} (no shards)")
        return out

    def _read_piece(self, shard: int, b: TensorBuilder) -> np.ndarray:
        """rows x cols f16 bits of one shard's piece, read row by row like src/tensor.rs:2452-2480."""
        if b.stride < 1:
            raise ValueError(f"invalid stride {b.stride}")
        # The pickle is untrusted input (BININT / BININT2 are signed): check every extent before it sizes a read, and
        # take the storage key only as a file name inside consolidated.NN/data/ (src/data_source.rs:105-111).
        if b.rows <= 0 or b.cols <= 0 or b.offset < 0 or b.nitems < 0 or b.offset + b.rows * b.cols > b.nitems:
            raise ValueError(f"{b.tensor_name}: shape {b.rows}x{b.cols} at offset {b.offset} does not fit its storage of {b.nitems} items")
        if not b.src_path or "/" in b.src_path or "\\" in b.src_path or b.src_path in (".", ".."):
            raise ValueError(f"{b.tensor_name}: storage key {b.src_path!r} is not a plain file name")
        fn = os.path.join(self.path, f"consolidated.{shard:02d}", "data", b.src_path)
        want = b.rows * b.cols
        arr = np.fromfile(fn, dtype="<u2", count=want, offset=2 * b.offset)
        if arr.size != want:
            raise IOError(f"path={fn} expected {want} items at offset {b.offset}, file holds {arr.size}")
        return arr.reshape(b.rows, b.cols)

    def load_f16_bits(self, name: str, direction: str, first_only: bool = False) -> np.ndarray:
        """TensorBuilder::load_from_pieces (src/tensor.rs:2391-2546) without the conversion to f32."""
        bs = self._builders(name, first_only)
        pieces = [self._read_piece(i, b) for i, b in enumerate(bs)]
        if direction == FROM_PIECES_ROWS:
            if any(p.shape[1] != pieces[0].shape[1] for p in pieces):
                raise ValueError(f"{name}: pieces differ in cols")
            return np.ascontiguousarray(np.concatenate(pieces, axis=0))
        if any(p.shape[0] != pieces[0].shape[0] for p in pieces):
            raise ValueError(f"{name}: pieces differ in rows")
        return np.ascontiguousarray(np.concatenate(pieces, axis=1))


# which tensor goes where: (name format, direction, first shard only); src/transformer.rs:297-304, 405-412, 490-503, 595-614
_TOP = {"tok_embeddings": ("tok_embeddings.weight", FROM_PIECES_COLS, False), "norm": ("norm.weight", FROM_PIECES_ROWS, True),
        "output": ("output.weight", FROM_PIECES_ROWS, False)}
_LAYER = {"wq": ("layers.{}.attention.wq.weight", FROM_PIECES_ROWS, False), "wk": ("layers.{}.attention.wk.weight", FROM_PIECES_ROWS, False),
          "wv": ("layers.{}.attention.wv.weight", FROM_PIECES_ROWS, False), "wo": ("layers.{}.attention.wo.weight", FROM_PIECES_COLS, False),
          "w1": ("layers.{}.feed_forward.w1.weight", FROM_PIECES_ROWS, False), "w2": ("layers.{}.feed_forward.w2.weight", FROM_PIECES_COLS, False),
          "w3": ("layers.{}.feed_forward.w3.weight", FROM_PIECES_ROWS, False),
          "attention_norm": ("layers.{}.attention_norm.weight", FROM_PIECES_ROWS, True), "ffn_norm": ("layers.{}.ffn_norm.weight", FROM_PIECES_ROWS, True)}


def load_transformer(ctx, model_path: str, data_settings, max_seq_len: int):
    """main's model construction (src/rllama_main.rs:235-283) + Transformer::from_unpickled (src/transformer.rs:242-326):
    reads every tensor of the directory that belongs on the device and hands its f16 bits to the device model (the values
    the reference gets after its f16 -> f32 -> f16 round trip are the same bits)."""
    import rllama_amd as ra

    ck = Checkpoint(model_path)
    w1 = ck._builders(_LAYER["w1"][0].format(0), False)
    ffn = sum(b.rows for b in w1)  # the FFN width is only in the stored shape
    tr = ra.Transformer(ctx, ck.dim, ck.n_layers, ck.n_heads, ffn, ck.vocab_size, max_seq_len, ck.norm_eps, data_settings)
    kinds = {"tok_embeddings": ra.TOK_EMB, "norm": ra.NORM, "output": ra.OUTPUT, "wq": ra.WQ, "wk": ra.WK, "wv": ra.WV, "wo": ra.WO,
             "w1": ra.W1, "w2": ra.W2, "w3": ra.W3, "attention_norm": ra.ATTN_NORM, "ffn_norm": ra.FFN_NORM}
    # With percentage_to_gpu below 1 only the leading layers live on the device (src/transformer.rs:262-279); the other
    # blocks, the embedding table and the output head are the host's (it reads them with Checkpoint.load_f16_bits itself).
    last = tr.last_layer_on_gpu()
    whole = last == ck.n_layers - 1
    for key, (name, direction, first) in _TOP.items():
        if whole or key == "norm":
            tr.set_tensor(kinds[key], 0, ck.load_f16_bits(name, direction, first))
    for l in range(last + 1):
        for key, (fmt, direction, first) in _LAYER.items():
            tr.set_tensor(kinds[key], l, ck.load_f16_bits(fmt.format(l), direction, first))
    return tr


# ---------------------------------------------------------------------------------------------------------------
# writer: the smallest data.pkl the reference's unpickler accepts (and CPython's pickle reads the same way)


def _binunicode(s: str) -> bytes:
    b = s.encode("utf-8")
    return b"\x58" + struct.pack("<I", len(b)) + b


def _binint(v: int) -> bytes:
    # always the 4-byte form: the reference reads BININT2 as signed (src/unpickler.rs:484)
    return b"\x4a" + struct.pack("<i", v)


def pickle_state_dict(entries: Sequence[Tuple[str, str, Tuple[int, ...]]]) -> bytes:
    """entries: (tensor name, storage key, shape[, storage offset, storage items]).  One dict, one MARK ... SETITEMS batch.
    The two optional fields default to 0 and the shape's element count (tests use them to write damaged files)."""
    out = bytearray(b"\x80\x02\x7d\x28")
    for name, key, shape, *rest in entries:
        if len(shape) not in (1, 2):
            raise ValueError("only 1-D and 2-D tensors")
        offset = int(rest[0]) if len(rest) > 0 else 0
        nitems = int(rest[1]) if len(rest) > 1 else int(np.prod(shape))
        out += _binunicode(name)
        out += b"ctorch._utils\n_rebuild_tensor_v2\n"
        out += b"\x28"                                             # MARK: args tuple
        out += b"\x28" + _binunicode("storage") + b"ctorch\nHalfStorage\n" + _binunicode(key) + _binunicode("cpu") + _binint(nitems) + b"\x74"
        out += b"\x51"                                             # BINPERSID
        out += _binint(offset)                                     # storage offset
        if len(shape) == 2:
            out += _binint(shape[0]) + _binint(shape[1]) + b"\x86" + _binint(shape[1]) + _binint(1) + b"\x86"
        else:
            out += _binint(shape[0]) + b"\x85" + _binint(1) + b"\x85"
        out += b"\x89"                                             # requires_grad = False
        out += b"ccollections\nOrderedDict\n\x29\x52"               # backward hooks: OrderedDict()
        out += b"\x74\x52"                                         # TUPLE, REDUCE
    out += b"\x75\x2e"                                             # SETITEMS, STOP
    return bytes(out)


def write_checkpoint(model_path: str, params: dict, tensors: Dict[str, np.ndarray], n_shards: int = 1) -> None:
    """Writes params.json and consolidated.NN/{data.pkl,data/<k>}.  `tensors` maps the reference's names to uint16
    (f16 bits) arrays, 1-D or 2-D.  With n_shards > 1 every matrix is split the way the reference joins it
    (rows or columns, see _TOP / _LAYER); norm weights are repeated in every shard."""
    os.makedirs(model_path, exist_ok=True)
    with open(os.path.join(model_path, "params.json"), "w") as f:
        json.dump(params, f)
    direction = {}
    for name in tensors:
        base = name
        parts = name.split(".")
        if parts[0] == "layers":
            base = "layers.{}." + ".".join(parts[2:])
        d = None
        for fmt, dirn, first in list(_TOP.values()) + list(_LAYER.values()):
            if fmt == base:
                d = (dirn, first)
        if d is None:
            raise KeyError(f"unknown tensor name {name}")
        direction[name] = d
    for s in range(n_shards):
        sd = os.path.join(model_path, f"consolidated.{s:02d}")
        os.makedirs(os.path.join(sd, "data"), exist_ok=True)
        entries = []
        for k, (name, arr) in enumerate(tensors.items()):
            if arr.dtype != np.uint16:
                raise TypeError(f"{name}: expected f16 bits (uint16)")
            dirn, first = direction[name]
            piece = arr
            if n_shards > 1 and not first:
                axis = 0 if dirn == FROM_PIECES_ROWS else 1
                if arr.ndim != 2 or arr.shape[axis] % n_shards:
                    raise ValueError(f"{name}: cannot split {arr.shape} into {n_shards} shards")
                piece = np.split(arr, n_shards, axis=axis)[s]
            piece = np.ascontiguousarray(piece)
            piece.astype("<u2").tofile(os.path.join(sd, "data", str(k)))
            entries.append((name, str(k), tuple(int(v) for v in piece.shape)))
        with open(os.path.join(sd, "data.pkl"), "wb") as f:
            f.write(pickle_state_dict(entries))


def write_synthetic_checkpoint(model_path: str, dim: int = 1024, n_layers: int = 8, n_heads: int = 16, ffn_hidden: int = 2816, vocab_size: int = 32000,
                               norm_eps: float = 1e-6, seed: int = 0, std: float = 0.02, n_shards: int = 1) -> None:
    """The benchmark's synthetic model (weights N(0, std) from the counter-based generator, norm weights 1.0) as a model
    directory the reference can be pointed at (--model-path; it also wants a tokenizer model, which this does not make).
    The defaults are config 0."""
    import rllama_amd as ra

    one = np.full(dim, 0x3C00, dtype=np.uint16)  # 1.0 in f16
    T: Dict[str, np.ndarray] = {}

    def gen(kind, layer, rows, cols):
        return ra.synth_normal_f16(seed, kind, layer, rows * cols, std=std).reshape(rows, cols)

    T["tok_embeddings.weight"] = gen(ra.TOK_EMB, 0, vocab_size, dim)
    T["norm.weight"] = one
    T["output.weight"] = gen(ra.OUTPUT, 0, vocab_size, dim)
    for l in range(n_layers):
        p = f"layers.{l}."
        for nm, kind in (("attention.wq", ra.WQ), ("attention.wk", ra.WK), ("attention.wv", ra.WV), ("attention.wo", ra.WO)):
            T[p + nm + ".weight"] = gen(kind, l, dim, dim)
        T[p + "feed_forward.w1.weight"] = gen(ra.W1, l, ffn_hidden, dim)
        T[p + "feed_forward.w2.weight"] = gen(ra.W2, l, dim, ffn_hidden)
        T[p + "feed_forward.w3.weight"] = gen(ra.W3, l, ffn_hidden, dim)
        T[p + "attention_norm.weight"] = one
        T[p + "ffn_norm.weight"] = one
    write_checkpoint(model_path, {"dim": dim, "multiple_of": 256, "n_heads": n_heads, "n_layers": n_layers, "norm_eps": norm_eps, "vocab_size": vocab_size},
                     T, n_shards=n_shards)


if __name__ == "__main__":
    import argparse

    ap = argparse.ArgumentParser(description="write the synthetic benchmark model (default: config 0) in the reference's on-disk layout")
    ap.add_argument("model_path")
    for name, default in (("dim", 1024), ("n-layers", 8), ("n-heads", 16), ("ffn-hidden", 2816), ("vocab-size", 32000), ("seed", 0), ("shards", 1)):
        ap.add_argument("--" + name, type=int, default=default)
    a = ap.parse_args()
    write_synthetic_checkpoint(a.model_path, a.dim, a.n_layers, a.n_heads, a.ffn_hidden, a.vocab_size, seed=a.seed, n_shards=a.shards)
    print("wrote", a.model_path)
