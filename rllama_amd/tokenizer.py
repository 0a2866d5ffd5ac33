"""The reference's tokenizer (Noeda/rllama src/tokenizer.rs): reads a SentencePiece model file and tokenizes by naive
longest-prefix matching over its pieces.  This is NOT SentencePiece's own segmentation; it is what the reference does,
quirks included:

* a position where no piece matches is skipped one BYTE at a time, and if that lands inside a multi-byte character the
  rest of the text is dropped (`s.get(1..).unwrap_or("")`, src/tokenizer.rs:157-159);
* a newline becomes the byte piece `<0x0A>` when the model has one, and is dropped otherwise (:139-147);
* `tokenize_to_ids` puts "▁" in front, turns every space into "▁" and starts with id 1 (:166-177).

The model file is a protobuf (`ModelProto`, proto/sentencepiece_model.proto:282-321); only field 1 (the repeated
`SentencePiece {1: piece, 2: score, 3: type}`) is read, everything else is skipped by wire type.
"""
from __future__ import annotations

import struct
from typing import Dict, List, Optional, Tuple

# sentence_piece::Type (proto/sentencepiece_model.proto:284-293) -> PieceType (src/tokenizer.rs:16-24)
PIECE_TYPES = {1: "Normal", 2: "Unknown", 3: "Control", 4: "UserDefined", 6: "Byte", 5: "Unused"}


class TokenizerError(Exception):
    pass


def _varint(b: bytes, p: int) -> Tuple[int, int]:
    v, shift = 0, 0
    while True:
        if p >= len(b):
            raise TokenizerError("Protobuf error: truncated varint")
        c = b[p]
        p += 1
        v |= (c & 0x7F) << shift
        if not c & 0x80:
            return v, p
        shift += 7
        if shift > 63:
            raise TokenizerError("Protobuf error: varint too long")


def _fields(b: bytes):
    """Yields (field number, wire type, value) of one message; value is an int (varint, fixed) or bytes (length-delimited)."""
    p = 0
    while p < len(b):
        key, p = _varint(b, p)
        field, wt = key >> 3, key & 7
        if wt == 0:
            v, p = _varint(b, p)
        elif wt == 1:
            if p + 8 > len(b):
                raise TokenizerError("Protobuf error: truncated fixed64")
            v = struct.unpack_from("<Q", b, p)[0]
            p += 8
        elif wt == 2:
            ln, p = _varint(b, p)
            if p + ln > len(b):
                raise TokenizerError("Protobuf error: truncated field")
            v = b[p:p + ln]
            p += ln
        elif wt == 5:
            if p + 4 > len(b):
                raise TokenizerError("Protobuf error: truncated fixed32")
            v = struct.unpack_from("<I", b, p)[0]
            p += 4
        else:
            raise TokenizerError(f"Protobuf error: unsupported wire type {wt}")
        yield field, wt, v


class Tokenizer:
    def __init__(self, pieces: Dict[bytes, Tuple[str, float, int]]):
        # piece (UTF-8 bytes) -> (type, score, idx), kept in byte order like the reference's BTreeMap<String, Piece>
        self._pieces = dict(sorted(pieces.items()))

    @staticmethod
    def load(path: str) -> "Tokenizer":
        with open(path, "rb") as f:
            return Tokenizer.from_bytes(f.read())

    @staticmethod
    def from_bytes(model: bytes) -> "Tokenizer":
        """Tokenizer::load (src/tokenizer.rs:45-95)."""
        pieces: Dict[bytes, Tuple[str, float, int]] = {}
        idx = 0
        for field, wt, v in _fields(model):
            if field != 1 or wt != 2:
                continue
            piece: Optional[bytes] = None
            score = 0.0
            tp = 1  # default NORMAL
            for f2, wt2, v2 in _fields(v):
                if f2 == 1 and wt2 == 2:
                    piece = v2
                elif f2 == 2 and wt2 == 5:
                    score = struct.unpack("<f", struct.pack("<I", v2))[0]
                elif f2 == 3 and wt2 == 0:
                    tp = v2
            if piece is not None:  # a piece without a string is skipped but still counts for the ids (:52-57)
                try:
                    piece.decode("utf-8")
                except UnicodeDecodeError as e:
                    raise TokenizerError("Protobuf error: piece is not UTF-8") from e
                if tp not in PIECE_TYPES:
                    raise TokenizerError(f"Unknown piece type: {piece.decode('utf-8')}")
                pieces[piece] = (PIECE_TYPES[tp], score, idx)  # a repeated string keeps the later entry (BTreeMap::insert)
            idx += 1
        return Tokenizer(pieces)

    def __len__(self) -> int:
        return len(self._pieces)

    def id_to_str(self, id: int) -> str:
        """Panics (IndexError here) if no piece carries this id (:99-107)."""
        for s, (_, _, idx) in self._pieces.items():
            if idx == id:
                return s.decode("utf-8")
        raise IndexError("id out of range")

    def str_to_id(self, s: str) -> Optional[int]:
        e = self._pieces.get(s.encode("utf-8"))
        return None if e is None else e[2]

    def piece_info(self, s: str) -> Optional[Tuple[str, float, int]]:
        return self._pieces.get(s.encode("utf-8"))

    def tokenize_to_pieces(self, text: str) -> List[str]:
        """src/tokenizer.rs:127-164."""
        s = text.encode("utf-8")
        out: List[str] = []
        have_nl = b"<0x0A>" in self._pieces
        while s:
            best: Optional[bytes] = None
            rest = b""
            if s[0] == 0x0A:
                if have_nl:
                    best, rest = b"<0x0A>", s[1:]
                # else: the candidate "\\n" has length 0 in the reference, so the byte is skipped below
            else:
                best_len = 0
                for piece in self._pieces:
                    if len(piece) > best_len and s.startswith(piece):
                        best, best_len, rest = piece, len(piece), s[len(piece):]
            if best is None:
                # skip one byte; when that is not a character boundary the reference's str::get returns None and the
                # remaining text becomes empty
                s = s[1:] if len(s) > 1 and (s[1] & 0xC0) != 0x80 else b""
            else:
                out.append(best.decode("utf-8"))
                s = rest
        return out

    def tokenize_to_ids(self, text: str) -> List[int]:
        """src/tokenizer.rs:166-177: "▁" + text with spaces turned into "▁", ids preceded by the start token 1."""
        s = ("▁" + text).replace(" ", "▁")
        return [1] + [self._pieces[p.encode("utf-8")][2] for p in self.tokenize_to_pieces(s)]
