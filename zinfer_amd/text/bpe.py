"""Byte-level BPE as the reference applies it (`src/tokenizer/bpe.zig`, `src/tokenizer/bpe/`).

Encoding (`bpe.zig:65-87`): at every offset the longest special token wins
(`bpe/pretokenize.zig:4-14`); otherwise one pre-token is cut by hand-written rules
(`pretokenize.zig:16-158`), its bytes go through the byte -> code point table
(`bpe/byte_mapping.zig:13-44`), neighbouring pieces are merged lowest rank first
(`bpe/merge.zig:17-34`) and the pieces are looked up in the vocabulary (`bpe.zig:135-138`).
Decoding (`bpe.zig:89-118`): token strings are concatenated, code points go back to bytes
except for special tokens, which are written as they are, and bytes that are no UTF-8 become
U+FFFD (`bpe.zig:154-176`).

Files: ``tokenizer.json`` (``model.vocab``, ``model.merges``, ``added_tokens``) when the folder
has one, else the reference's three files ``vocab.json``, ``merges.txt`` and
``tokenizer_config.json`` (``added_tokens_decoder``) (`bpe.zig:23-63`, `bpe/io.zig`).
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional, Sequence, Tuple

from ..errors import ZinferError


class TokenizerError(ZinferError):
    """TokenizerNotFound, InvalidVocab, InvalidTokenizerConfig, TokenNotFound, UnknownTokenId."""


def byte_table() -> Tuple[List[str], Dict[str, int]]:
    """Byte -> one printable code point and back: '!'..'~', 0xA1..0xAC and 0xAE..0xFF stand
    for themselves, the other 68 bytes take 256, 257, ... in ascending byte order
    (`bpe/byte_mapping.zig:13-44`)."""
    keep = list(range(ord("!"), ord("~") + 1)) + list(range(0xA1, 0xAD)) + list(range(0xAE, 0x100))
    encoder: List[Optional[str]] = [None] * 256
    for b in keep:
        encoder[b] = chr(b)
    extra = 0
    for b in range(256):
        if encoder[b] is None:
            encoder[b] = chr(256 + extra)
            extra += 1
    return encoder, {c: b for b, c in enumerate(encoder)}


# ----------------------------------------------------------------------------- pre-tokens
def _is_space(c: str) -> bool:            # `pretokenize.zig:170-175`
    return c == " " or c == "\t"


def _is_newline(c: str) -> bool:          # `:177-179`
    return c == "\n" or c == "\r"


def _is_digit(c: str) -> bool:            # `:181-183`
    return "0" <= c <= "9"


def _is_punctuation_block(cp: int) -> bool:   # `:196-207`
    return (0x2000 <= cp <= 0x206F or 0x3000 <= cp <= 0x303F or 0xFF00 <= cp <= 0xFF0F
            or 0xFF1A <= cp <= 0xFF20 or 0xFF3B <= cp <= 0xFF40 or 0xFF5B <= cp <= 0xFF65)


def _is_letter(c: str) -> bool:           # `:185-194`
    cp = ord(c)
    if cp < 128:
        return ("a" <= c <= "z") or ("A" <= c <= "Z")
    if (0x4E00 <= cp <= 0x9FFF or 0x3400 <= cp <= 0x4DBF or 0x3040 <= cp <= 0x30FF
            or 0xAC00 <= cp <= 0xD7AF or 0x0400 <= cp <= 0x052F or 0x00C0 <= cp <= 0x024F):
        return True
    return not _is_space(c) and not _is_newline(c) and not _is_punctuation_block(cp)


_CONTRACTIONS = ("'s", "'t", "'re", "'ve", "'m", "'ll", "'d")     # `:160-168`


class _Cutter:
    """Cuts one pre-token at a time; a special token ends every run (`pretokenize.zig`)."""

    def __init__(self, text: str, specials: Sequence[str]):
        self.text, self.specials = text, specials

    def special_at(self, i: int) -> Optional[str]:
        best = None
        for s in self.specials:
            if self.text.startswith(s, i) and (best is None or len(s) > len(best)):
                best = s
        return best

    def _run(self, i: int, keep) -> int:
        """End of the run of characters satisfying ``keep`` from ``i`` on."""
        t = self.text
        while i < len(t) and self.special_at(i) is None and keep(t[i]):
            i += 1
        return i

    def _punctuation_from(self, i: int) -> int:
        """A punctuation run and the newlines right after it (`:84-103,138-156`)."""
        i = self._run(i, lambda c: not (_is_digit(c) or _is_letter(c) or _is_newline(c) or _is_space(c)))
        return self._run(i, _is_newline)

    def next(self, start: int) -> int:
        """The end of the pre-token that begins at ``start`` (which holds no special token)."""
        t = self.text
        first = t[start]
        if _is_newline(first):                                       # `:24-36`
            return self._run(start + 1, _is_newline)
        if _is_space(first):                                         # `:38-108`
            end = self._run(start, _is_space)
            if end < len(t) and self.special_at(end) is None:
                c = t[end]
                if _is_letter(c):
                    # all spaces but the last stand alone; the last one goes with the word
                    if end - start > 1:
                        return end - 1
                    return self._run(end + 1, _is_letter)
                if not _is_digit(c) and not _is_newline(c) and not _is_space(c):
                    if end - start > 1:
                        return end - 1
                    return self._punctuation_from(end + 1)
            return end
        if first == "'":                                             # `:110-115`
            for item in _CONTRACTIONS:
                if t[start:start + len(item)].lower() == item:
                    return start + len(item)
        if _is_letter(first):                                        # `:117-129`
            return self._run(start + 1, _is_letter)
        if _is_digit(first):                                         # `:131-143`: runs of any length
            return self._run(start + 1, _is_digit)
        return self._punctuation_from(start + 1)                     # `:145-157`


def pre_tokens(text: str, specials: Sequence[str]) -> List[Tuple[str, bool]]:
    """(piece, is_special) in order; the pieces concatenate to ``text``."""
    cutter = _Cutter(text, specials)
    out: List[Tuple[str, bool]] = []
    i = 0
    while i < len(text):
        s = cutter.special_at(i)
        if s is not None:
            out.append((s, True))
            i += len(s)
            continue
        end = cutter.next(i)
        out.append((text[i:end], False))
        i = end
    return out


# ----------------------------------------------------------------------------- the tokenizer
class Tokenizer:
    def __init__(self, vocab: Dict[str, int], merges: Sequence[str], specials: Dict[str, int]):
        """``vocab``: token string (in the byte alphabet) -> id; ``merges``: "left right" in
        rank order; ``specials``: content -> id, matched on the raw text."""
        self.vocab = dict(vocab)
        self.specials = dict(specials)
        for content, tid in self.specials.items():
            self.vocab[content] = tid                       # `bpe/io.zig:65`
        self.ranks = {}
        for line in merges:
            line = line.strip(" \r\t")
            if not line or line.startswith("#"):            # `bpe/io.zig:32-40`
                continue
            self.ranks.setdefault(line, len(self.ranks))
        self.special_ids = set(self.specials.values())
        # longest first (`bpe/io.zig:72-76`)
        self._special_list = sorted(self.specials, key=len, reverse=True)
        self.id_to_token: Dict[int, str] = {i: s for s, i in self.vocab.items()}
        self._enc, self._dec = byte_table()

    # ------------------------------------------------------------------ loading
    @classmethod
    def from_dir(cls, model_dir: str) -> "Tokenizer":
        tj = os.path.join(model_dir, "tokenizer.json")
        if os.path.exists(tj):
            with open(tj, "r", encoding="utf-8") as f:
                raw = json.load(f)
            model = raw.get("model")
            if not isinstance(model, dict) or not isinstance(model.get("vocab"), dict):
                raise TokenizerError("InvalidVocab: tokenizer.json has no model.vocab object")
            merges = []
            for m in model.get("merges", []):
                merges.append(m if isinstance(m, str) else " ".join(m))
            specials = {}
            for t in raw.get("added_tokens", []):
                if not isinstance(t, dict) or "content" not in t or "id" not in t:
                    raise TokenizerError("InvalidTokenizerConfig: added_tokens entries need id and content")
                specials[str(t["content"])] = int(t["id"])
            return cls(_checked_vocab(model["vocab"]), merges, specials)
        vj = os.path.join(model_dir, "vocab.json")
        mt = os.path.join(model_dir, "merges.txt")
        tc = os.path.join(model_dir, "tokenizer_config.json")
        if not (os.path.exists(vj) and os.path.exists(mt)):
            raise TokenizerError(f"TokenizerNotFound: {model_dir} has neither tokenizer.json nor "
                                 "vocab.json + merges.txt")
        with open(vj, "r", encoding="utf-8") as f:
            vocab = _checked_vocab(json.load(f))
        with open(mt, "r", encoding="utf-8") as f:
            merges = f.read().split("\n")
        specials = {}
        if os.path.exists(tc):
            with open(tc, "r", encoding="utf-8") as f:
                cfg = json.load(f)
            dec = cfg.get("added_tokens_decoder") if isinstance(cfg, dict) else None
            if not isinstance(dec, dict):
                raise TokenizerError("InvalidTokenizerConfig: no added_tokens_decoder object")
            for key, val in dec.items():                    # `bpe/io.zig:58-70`
                if not isinstance(val, dict) or not isinstance(val.get("content"), str):
                    raise TokenizerError("InvalidTokenizerConfig: added_tokens_decoder entry without content")
                specials[val["content"]] = int(key)
        return cls(vocab, merges, specials)

    @staticmethod
    def present(model_dir: str) -> bool:
        return os.path.exists(os.path.join(model_dir, "tokenizer.json")) or (
            os.path.exists(os.path.join(model_dir, "vocab.json"))
            and os.path.exists(os.path.join(model_dir, "merges.txt")))

    # ------------------------------------------------------------------ encode / decode
    def _merge(self, symbols: List[str]) -> List[str]:
        """Lowest rank first, leftmost among equals, one pair at a time (`merge.zig:17-34`)."""
        pieces = list(symbols)
        while len(pieces) >= 2:
            best, at = None, 0
            for i in range(len(pieces) - 1):
                rank = self.ranks.get(pieces[i] + " " + pieces[i + 1])
                if rank is not None and (best is None or rank < best):
                    best, at = rank, i
            if best is None:
                break
            pieces[at:at + 2] = [pieces[at] + pieces[at + 1]]
        return pieces

    def encode(self, text: str) -> List[int]:
        ids: List[int] = []
        for piece, special in pre_tokens(text, self._special_list):
            if special:
                ids.append(self.specials[piece])
                continue
            symbols = [self._enc[b] for b in piece.encode("utf-8")]
            for token in self._merge(symbols):
                tid = self.vocab.get(token)
                if tid is None:
                    raise TokenizerError(f"TokenNotFound: {token!r}")
                ids.append(tid)
        return ids

    def decode_bytes(self, ids: Sequence[int]) -> bytes:
        out = bytearray()
        for tid in ids:
            token = self.id_to_token.get(int(tid))
            if token is None:
                raise TokenizerError(f"UnknownTokenId: {tid}")
            if int(tid) in self.special_ids:
                out += token.encode("utf-8")
                continue
            for c in token:
                b = self._dec.get(c)
                if b is None:
                    raise TokenizerError(f"InvalidByteDecoderEntry: {c!r} in token {tid}")
                out.append(b)
        return bytes(out)

    def decode(self, ids: Sequence[int]) -> str:
        return utf8_lossy(self.decode_bytes(ids))


def _checked_vocab(raw) -> Dict[str, int]:
    if not isinstance(raw, dict):
        raise TokenizerError("InvalidVocab: the vocabulary must be an object of token -> id")
    for k, v in raw.items():
        if not isinstance(v, int) or isinstance(v, bool):
            raise TokenizerError(f"InvalidVocab: id of {k!r} is not an integer")
    return raw


def utf8_lossy(raw: bytes) -> str:
    """Valid sequences as they are; every byte that starts none becomes U+FFFD
    (`bpe.zig:154-176`)."""
    try:
        return raw.decode("utf-8")
    except UnicodeDecodeError:
        pass
    out: List[str] = []
    i = 0
    while i < len(raw):
        b = raw[i]
        n = 1 if b < 0x80 else 2 if 0xC0 <= b < 0xE0 else 3 if 0xE0 <= b < 0xF0 else \
            4 if 0xF0 <= b < 0xF8 else 0
        if n and i + n <= len(raw):
            try:
                out.append(raw[i:i + n].decode("utf-8"))
                i += n
                continue
            except UnicodeDecodeError:
                pass
        out.append("�")
        i += 1
    return "".join(out)
