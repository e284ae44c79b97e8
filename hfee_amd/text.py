"""Text glue around the token ids: holding back bytes until they are valid UTF-8,
holding back text that may begin a stop string
(/root/reference/internal/llm/text.go:22-78), and a thin tokenizer over the folder's
tokenizer.json.  The engine itself deals in token ids only.
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


class FolderTokenizer:
    """tokenizer.json through the `tokenizers` library: text -> ids, id -> bytes."""

    def __init__(self, path: str):
        from tokenizers import Tokenizer
        self.tok = Tokenizer.from_file(path)

    def encode(self, text: str) -> list:
        return self.tok.encode(text, add_special_tokens=False).ids

    def piece(self, token: int) -> bytes:
        return self.tok.decode([token], skip_special_tokens=True).encode("utf-8")


def load_tokenizer(model_dir):
    path = os.path.join(model_dir, "tokenizer.json") if model_dir else None
    if path and os.path.isfile(path):
        return FolderTokenizer(path)
    return None
