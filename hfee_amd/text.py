"""Text glue around the token ids: holding back bytes until they are valid UTF-8,
holding back text that may begin a stop string
(/root/reference/internal/llm/text.go:22-78), and the tokenizer over the folder's
tokenizer.json (the reference's rules, /root/reference/internal/tokenizer).  The engine
itself deals in token ids only.
"""
from __future__ import annotations

import os


class Utf8Buffer:
    """Collects token bytes and releases the longest prefix that is complete UTF-8."""

    def __init__(self):
        self.pending = b""

    def add(self, piece: bytes) -> str:
        data = self.pending + piece
        cut = len(data)
        # step back over an incomplete trailing sequence (at most 3 bytes)
        for back in range(1, min(4, len(data)) + 1):
            b = data[-back]
            if b & 0xC0 == 0x80:
                continue                       # continuation byte: keep looking for the lead
            need = 1 if b < 0x80 else 2 if b >> 5 == 0b110 else 3 if b >> 4 == 0b1110 else 4 if b >> 3 == 0b11110 else 1
            if need > back:
                cut = len(data) - back
            break
        self.pending = data[cut:]
        return data[:cut].decode("utf-8", errors="replace")

    def flush(self) -> str:
        out, self.pending = self.pending.decode("utf-8", errors="replace"), b""
        return out


class Stopper:
    """Passes text through, holding back any tail that could begin a stop string."""

    def __init__(self, stops):
        self.stops = [s for s in stops if s]
        self.held = ""

    def push(self, text: str):
        """-> (text safe to emit, whether a stop string was hit)."""
        if not self.stops:
            return text, False
        self.held += text
        for s in self.stops:
            i = self.held.find(s)
            if i >= 0:
                out, self.held = self.held[:i], ""
                return out, True
        keep = 0
        for s in self.stops:
            for k in range(min(len(s) - 1, len(self.held)), 0, -1):
                if self.held.endswith(s[:k]):
                    keep = max(keep, k)
                    break
        cut = len(self.held) - keep
        out, self.held = self.held[:cut], self.held[cut:]
        return out, False

    def flush(self) -> str:
        out, self.held = self.held, ""
        return out


# ------------------------------------------------------------------ tokenizer ---
# The reference's tokenizer (/root/reference/internal/tokenizer): text is cut at special
# tokens, which stay single ids (tokenizer.go:143-185); what lies between is cut into words
# by the rule the model was trained with (pretokenize.go), every word's bytes are written as
# printable characters (tokenizer.go:264-283), and adjacent pieces are joined, lowest merge
# rank first, leftmost first among equals, until no known pair is left (merge.go:7-60).  The
# reference reads vocabulary and merges from a GGUF file; here they come from the model
# folder's tokenizer.json.

def _byte_alphabet():
    """GPT-2's reversible map from bytes to printable characters (tokenizer.go:264-283):
    printable bytes stand for themselves, the others take the code points from 256 on."""
    forward, n = {}, 0
    for b in range(256):
        printable = 0x21 <= b <= 0x7E or 0xA1 <= b <= 0xAC or 0xAE <= b <= 0xFF
        forward[b] = chr(b) if printable else chr(256 + n)
        n += 0 if printable else 1
    return forward, {c: b for b, c in forward.items()}


_BYTE_TO_CHAR, _CHAR_TO_BYTE = _byte_alphabet()


def _is_letter(c: str) -> bool:
    import unicodedata
    return unicodedata.category(c)[0] == "L"


def _is_number(c: str) -> bool:
    import unicodedata
    return unicodedata.category(c)[0] == "N"


def _is_space(c: str) -> bool:
    import unicodedata
    return c in "\t\n\v\f\r \x85\xa0" or unicodedata.category(c) in ("Zs", "Zl", "Zp")


def _is_newline(c: str) -> bool:
    return c == "\r" or c == "\n"


def _is_symbol(c: str) -> bool:
    return not (_is_space(c) or _is_letter(c) or _is_number(c))


def _run(text: str, i: int, belongs) -> int:
    while i < len(text) and belongs(text[i]):
        i += 1
    return i


def _contraction(text: str, i: int, fold: bool) -> int:
    """End of 's 't 're 've 'm 'll 'd at i, or -1 (pretokenize.go:43-66)."""
    if text[i] != "'" or i + 1 >= len(text):
        return -1
    tail = text[i + 1:i + 3]
    if fold:
        tail = tail.lower()
    if tail[:1] in ("s", "t", "m", "d"):
        return i + 2
    return i + 3 if tail in ("re", "ve", "ll") else -1


def _spaces(text: str, i: int) -> int:
    """\\s+(?!\\S), else \\s+: a run of spaces gives up its last one to the word that follows
    (pretokenize.go:68-75)."""
    end = _run(text, i, _is_space)
    return end - 1 if end < len(text) and end - i > 1 else end


def split_llama3(text: str, max_digits: int = 3) -> list:
    """The words of (?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\\r\\n\\p{L}\\p{N}]?\\p{L}+|\\p{N}{1,n}|
     ?[^\\s\\p{L}\\p{N}]+[\\r\\n]*|\\s*[\\r\\n]+|\\s+(?!\\S)|\\s+, alternative by alternative as the
    reference walks them (pretokenize.go:77-127)."""
    out, i = [], 0
    while i < len(text):
        c = text[i]
        end = _contraction(text, i, True)
        if end < 0:
            lead = i + 1 if (not _is_letter(c) and not _is_number(c) and not _is_newline(c)
                             and i + 1 < len(text) and _is_letter(text[i + 1])) else i
            if _is_letter(text[lead]):
                end = _run(text, lead, _is_letter)
            elif _is_number(c):
                end = i
                while end < len(text) and end - i < max_digits and _is_number(text[end]):
                    end += 1
            else:
                start = i + 1 if c == " " else i
                if start < len(text) and _is_symbol(text[start]):
                    end = _run(text, _run(text, start, _is_symbol), _is_newline)
                elif _is_space(c):
                    stop = _run(text, i, _is_space)
                    last_newline = max((k for k in range(i, stop) if _is_newline(text[k])), default=-1)
                    end = last_newline + 1 if last_newline >= 0 else _spaces(text, i)
                else:
                    end = i + 1
        out.append(text[i:end])
        i = end
    return out


def split_gpt2(text: str) -> list:
    """'s|'t|'re|'ve|'m|'ll|'d| ?\\p{L}+| ?\\p{N}+| ?[^\\s\\p{L}\\p{N}]+|\\s+(?!\\S)|\\s+
    (pretokenize.go:129-148)."""
    out, i = [], 0
    while i < len(text):
        end = _contraction(text, i, False)
        if end < 0:
            start = i + 1 if text[i] == " " else i
            kind = next((k for k in (_is_letter, _is_number, _is_symbol) if start < len(text) and k(text[start])), None)
            if kind is not None:
                end = _run(text, start, kind)
            elif _is_space(text[i]):
                end = _spaces(text, i)
            else:
                end = i + 1
        out.append(text[i:end])
        i = end
    return out


def merge_pieces(pieces: list, rank) -> list:
    """Joins the adjacent pair with the lowest rank, the leftmost one among equals, until
    `rank(left, right)` (a number, or None for a pair that is not known) knows none of the
    pairs left (merge.go:7-60)."""
    pieces = list(pieces)
    while len(pieces) > 1:
        best, where = None, -1
        for k in range(len(pieces) - 1):
            r = rank(pieces[k], pieces[k + 1])
            if r is not None and (best is None or r < best):
                best, where = r, k
        if where < 0:
            break
        pieces[where:where + 2] = [pieces[where] + pieces[where + 1]]
    return pieces


class FolderTokenizer:
    """A model folder's tokenizer.json: text -> ids, id -> bytes.  Byte-level vocabularies
    (words cut by the llama3 or the gpt2 rule, bytes written as printable characters) and
    vocabularies of the sentencepiece kind (spaces written as U+2581, bytes without a piece
    as <0xNN>) are read; the merges' order is their rank.  (The reference joins the pieces of a
    sentencepiece vocabulary by the scores in its model file, tokenizer.go:185-212; a
    tokenizer.json has none, and its merges are taken to be in descending score, as the
    converters write them.  A piece without an id and without byte pieces is dropped, as there.)"""

    def __init__(self, path: str):
        import json
        with open(path, "r", encoding="utf-8") as f:
            spec = json.load(f)
        model = spec.get("model") or {}
        if model.get("type", "BPE") != "BPE" or "vocab" not in model:
            raise ValueError(f"{path}: only tokenizers with a vocabulary and merges (type BPE) are read")
        self.vocab = dict(model["vocab"])
        self.ranks = {}
        for r, m in enumerate(model.get("merges") or []):
            left, right = m.split(" ", 1) if isinstance(m, str) else m
            self.ranks[(left, right)] = r
        self.pieces = {i: t for t, i in self.vocab.items()}
        self.special, self.control = {}, set()
        for a in spec.get("added_tokens") or []:
            self.special[a["content"]] = a["id"]
            self.pieces[a["id"]] = a["content"]
            if a.get("special", False):
                self.control.add(a["id"])
        parts = [spec.get("pre_tokenizer"), spec.get("decoder"), spec.get("normalizer")]
        kinds, patterns = set(), []

        def walk(node):
            if isinstance(node, dict):
                kinds.add(node.get("type"))
                pattern = node.get("pattern")
                if isinstance(pattern, dict):
                    patterns.append(str(pattern.get("Regex") or pattern.get("String") or ""))
                if node.get("add_prefix_space") is True or node.get("prepend_scheme") in ("first", "always"):
                    kinds.add("prefix")
                for v in node.values():
                    walk(v)
            elif isinstance(node, list):
                for v in node:
                    walk(v)

        walk(parts)
        self.byte_level = "ByteLevel" in kinds
        # the llama3 rule folds case in its contractions and takes digits one or three at a
        # time; anything else that is byte-level is cut by the gpt2 rule (pretokenize.go:20-41)
        self.llama3_rule = any("(?i:" in p for p in patterns)
        self.max_digits = 3 if any("{1,3}" in p for p in patterns) else 1
        self.space_prefix = not self.byte_level and ("Prepend" in kinds or "prefix" in kinds)
        self._by_first = {}
        for content in sorted(self.special, key=len, reverse=True):      # the longest special token at a place wins
            self._by_first.setdefault(content[0], []).append(content)
        self._word_cache = {}

    # ---- text -> ids
    def encode(self, text: str) -> list:
        """Special tokens written in the text stay single ids (tokenizer.go:143-185)."""
        ids, start, i, after_special = [], 0, 0, True
        while i < len(text):
            hit = next((t for t in self._by_first.get(text[i], ()) if text.startswith(t, i)), None)
            if hit is None:
                i += 1
                continue
            if i > start:
                ids += self._encode_plain(text[start:i], after_special)
            ids.append(self.special[hit])
            i += len(hit)
            start, after_special = i, True
        if start < len(text):
            ids += self._encode_plain(text[start:], after_special)
        return ids

    def _encode_plain(self, text: str, after_special: bool) -> list:
        if not self.byte_level:                                  # tokenizer.go:187-218
            if self.space_prefix and after_special:
                text = " " + text
            out = []
            for piece in merge_pieces(list(text.replace(" ", "\u2581")), lambda a, b: self.ranks.get((a, b))):
                if piece in self.vocab:
                    out.append(self.vocab[piece])
                else:
                    out += [self.vocab[f"<0x{b:02X}>"] for b in piece.encode("utf-8") if f"<0x{b:02X}>" in self.vocab]
            return out
        out = []
        words = split_llama3(text, self.max_digits) if self.llama3_rule else split_gpt2(text)
        for word in words:                                       # tokenizer.go:220-240
            ids = self._word_cache.get(word)
            if ids is None:
                symbols = [_BYTE_TO_CHAR[b] for b in word.encode("utf-8")]
                merged = merge_pieces(symbols, lambda a, b: self.ranks.get((a, b)))
                ids = [self.vocab[p] for p in merged if p in self.vocab]
                if len(self._word_cache) < 100000:
                    self._word_cache[word] = ids
            out += ids
        return out

    # ---- id -> bytes
    def piece(self, token: int) -> bytes:
        """The bytes a token stands for; control tokens stand for nothing (tokenizer.go:242-262).
        A token may hold part of a character only: the caller joins the bytes (Utf8Buffer)."""
        text = self.pieces.get(token)
        if text is None or token in self.control:
            return b""
        if token in self.special.values():
            return text.encode("utf-8")
        if self.byte_level:
            return bytes(_CHAR_TO_BYTE[c] for c in text if c in _CHAR_TO_BYTE)
        if len(text) == 6 and text.startswith("<0x") and text.endswith(">"):
            try:
                return bytes([int(text[3:5], 16)])
            except ValueError:
                pass
        return text.replace("\u2581", " ").encode("utf-8")


def load_tokenizer(model_dir):
    path = os.path.join(model_dir, "tokenizer.json") if model_dir else None
    if path and os.path.isfile(path):
        return FolderTokenizer(path)
    return None
