"""Tokenizers built from a GGUF file's own metadata (tokenizer.ggml.*), the two kinds llama.cpp writes:

  "llama"  SentencePiece-style vocabulary with a score per token: the text (spaces as U+2581, one in front) is cut into
           characters and the adjacent pair whose concatenation is the best-scoring token is merged until none is left;
           characters without a token fall back to the byte tokens <0xNN>;
  "gpt2"   byte-level BPE: the text is split by a pre-tokenizer pattern, bytes are mapped to printable characters and
           pairs are merged in the order of tokenizer.ggml.merges.

In the reference the tokenizer belongs to the third-party jitllm engine (jitnn-llm/.../llm/Llm.java:34-38 names it); these
are the published algorithms of the two vocabularies, enough to drive the generation loop end to end from a file.
"""
from __future__ import annotations

import heapq

SPACE = "▁"
TOKEN_NORMAL, TOKEN_UNKNOWN, TOKEN_CONTROL, TOKEN_USER, TOKEN_UNUSED, TOKEN_BYTE = 1, 2, 3, 4, 5, 6


def _byte_to_unicode() -> dict:
    """GPT-2's reversible map from bytes to printable code points."""
    keep = list(range(ord("!"), ord("~") + 1)) + list(range(0xA1, 0xAC + 1)) + list(range(0xAE, 0xFF + 1))
    table, extra = {}, 0
    for b in range(256):
        if b in keep:
            table[b] = chr(b)
        else:
            table[b] = chr(256 + extra)
            extra += 1
    return table


class Tokenizer:
    def __init__(self, model: str, tokens, scores=None, token_types=None, merges=None, bos=None, eos=None, add_bos=None, pre=None):
        if model not in ("llama", "gpt2"):
            raise ValueError(f"tokenizer model {model!r} (llama and gpt2 are built)")
        self.model, self.tokens = model, list(tokens)
        self.index = {}
        for i, t in enumerate(self.tokens):
            self.index.setdefault(t, i)
        self.scores = list(scores) if scores is not None else [0.0] * len(self.tokens)
        self.types = list(token_types) if token_types is not None else [TOKEN_NORMAL] * len(self.tokens)
        self.bos, self.eos = bos, eos
        self.add_bos = (model == "llama") if add_bos is None else bool(add_bos)
        self.pre = pre
        if model == "gpt2":
            self.ranks = {tuple(m.split(" ", 1)): r for r, m in enumerate(merges or [])}
            self.b2u = _byte_to_unicode()
            self.u2b = {u: b for b, u in self.b2u.items()}
        else:
            self.byte_token = {}
            for i, t in enumerate(self.tokens):
                if len(t) == 6 and t.startswith("<0x") and t.endswith(">") and (self.types[i] == TOKEN_BYTE or token_types is None):
                    try:
                        self.byte_token[int(t[3:5], 16)] = i
                    except ValueError:
                        pass
            self.unknown = next((i for i, ty in enumerate(self.types) if ty == TOKEN_UNKNOWN), 0)

    @staticmethod
    def from_gguf(f) -> "Tokenizer":
        """f: a jitnn_amd.GgufFile (or anything with has / string / strings / get)."""
        model = f.string("tokenizer.ggml.model")
        tokens = f.strings("tokenizer.ggml.tokens")
        scores = f.get("tokenizer.ggml.scores") if f.has("tokenizer.ggml.scores") else None
        types = f.get("tokenizer.ggml.token_type") if f.has("tokenizer.ggml.token_type") else None
        merges = f.strings("tokenizer.ggml.merges") if f.has("tokenizer.ggml.merges") else None
        geti = lambda k: int(f.get(k)) if f.has(k) else None
        add_bos = f.get("tokenizer.ggml.add_bos_token") if f.has("tokenizer.ggml.add_bos_token") else None
        pre = f.get("tokenizer.ggml.pre") if f.has("tokenizer.ggml.pre") else None
        return Tokenizer(model, tokens, scores, types, merges, geti("tokenizer.ggml.bos_token_id"), geti("tokenizer.ggml.eos_token_id"), add_bos, pre)

    # ---- text -> tokens
    def encode(self, text: str, add_bos: bool | None = None) -> list:
        ids = self._encode_spm(text) if self.model == "llama" else self._encode_bpe(text)
        if (self.add_bos if add_bos is None else add_bos) and self.bos is not None:
            ids = [self.bos] + ids
        return ids

    def _encode_spm(self, text: str) -> list:
        if not text:
            return []
        s = SPACE + text.replace(" ", SPACE)
        # doubly linked list of symbols; a heap of candidate merges (best score first, leftmost among equals)
        sym = list(s)
        prev = list(range(-1, len(sym) - 1))
        nxt = list(range(1, len(sym) + 1))
        nxt[-1] = -1
        heap = []

        def offer(left):
            right = nxt[left] if left >= 0 else -1
            if left < 0 or right < 0:
                return
            tok = self.index.get(sym[left] + sym[right])
            if tok is not None:
                heapq.heappush(heap, (-self.scores[tok], left, sym[left], sym[right]))

        for i in range(len(sym) - 1):
            offer(i)
        while heap:
            _, left, a, b = heapq.heappop(heap)
            right = nxt[left]
            if sym[left] is None or right < 0 or sym[left] != a or sym[right] != b:
                continue  # one of the two was merged away meanwhile
            sym[left] = a + b
            sym[right] = None
            nxt[left] = nxt[right]
            if nxt[right] >= 0:
                prev[nxt[right]] = left
            offer(prev[left])
            offer(left)
        out, i = [], 0
        while i >= 0:
            piece = sym[i]
            tok = self.index.get(piece)
            if tok is not None:
                out.append(tok)
            else:  # no token for this piece: its bytes, or the unknown token
                for b in piece.encode("utf-8"):
                    out.append(self.byte_token.get(b, self.unknown))
            i = nxt[i]
        return out

    def _split(self, text: str) -> list:
        import regex  # the pattern uses Unicode classes
        if self.pre in ("llama-bpe", "llama3", "llama-v3"):
            pat = (r"(?i:'s|'t|'re|'ve|'m|'ll|'d)|[^\r\n\p{L}\p{N}]?\p{L}+|\p{N}{1,3}| ?[^\s\p{L}\p{N}]+[\r\n]*|\s*[\r\n]+|\s+(?!\S)|\s+")
        else:  # GPT-2
            pat = r"'s|'t|'re|'ve|'m|'ll|'d| ?\p{L}+| ?\p{N}+| ?[^\s\p{L}\p{N}]+|\s+(?!\S)|\s+"
        return regex.findall(pat, text)

    def _encode_bpe(self, text: str) -> list:
        out = []
        for word in self._split(text):
            parts = [self.b2u[b] for b in word.encode("utf-8")]
            while len(parts) > 1:
                best, at = None, -1
                for i in range(len(parts) - 1):
                    r = self.ranks.get((parts[i], parts[i + 1]))
                    if r is not None and (best is None or r < best):
                        best, at = r, i
                if best is None:
                    break
                parts[at:at + 2] = [parts[at] + parts[at + 1]]
            for p in parts:
                tok = self.index.get(p)
                if tok is None:
                    raise ValueError(f"the vocabulary has no token for {p!r}")
                out.append(tok)
        return out

    # ---- tokens -> text
    def piece_bytes(self, tok: int) -> bytes:
        t = self.tokens[tok]
        if self.types[tok] == TOKEN_CONTROL:
            return b""
        if self.model == "llama":
            if self.types[tok] == TOKEN_BYTE or (tok in self.byte_token.values()):
                return bytes([int(t[3:5], 16)])
            return t.replace(SPACE, " ").encode("utf-8")
        return bytes(self.u2b.get(ch, ord("?")) for ch in t)

    def decode(self, ids, strip_leading_space: bool = False) -> str:
        s = b"".join(self.piece_bytes(i) for i in ids).decode("utf-8", "replace")
        return s[1:] if strip_leading_space and s.startswith(" ") else s


class StreamDecoder:
    """Turns a stream of token ids into pieces of text that add up to decode(all ids): bytes of a character that is split
    over tokens are held back until the character is whole."""

    def __init__(self, tok: Tokenizer):
        self.tok, self.pending = tok, b""

    def push(self, token: int) -> str:
        self.pending += self.tok.piece_bytes(token)
        for cut in range(len(self.pending), max(len(self.pending) - 4, -1), -1):
            try:
                s = self.pending[:cut].decode("utf-8")
            except UnicodeDecodeError:
                continue
            self.pending = self.pending[cut:]
            return s
        return ""

    def flush(self) -> str:
        s, self.pending = self.pending.decode("utf-8", "replace"), b""
        return s
