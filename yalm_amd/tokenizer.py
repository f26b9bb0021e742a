"""Text in and out, for the command line: the vocabulary of a folder's
tokenizer.json prepared as the reference's converter does (convert.py:86-125:
sentencepiece's U+2581 becomes a space, or the GPT-2 byte alphabet is mapped
back to bytes), greedy longest-match encoding over a trie with byte fallback
(src/tokenizer.cpp:57-94) and piece-by-piece decoding (src/tokenizer.cpp:44-55)."""
import json
import os


def _gpt2_byte_alphabet():
    """convert.py:84-96: the printable stand-ins of the 256 byte values."""
    bs = list(range(ord("!"), ord("~") + 1)) + list(range(0xA1, 0xAC + 1)) + list(range(0xAE, 0xFF + 1))
    cs = bs[:]
    n = 0
    for b in range(256):
        if b not in bs:
            bs.append(b)
            cs.append(256 + n)
            n += 1
    return {chr(c): b for b, c in zip(bs, cs)}


class Tokenizer:
    def __init__(self, vocab, bos_id, eos_id):
        self.vocab = vocab                       # list of bytes, index = token id
        self.bos_id = bos_id
        self.eos_id = eos_id
        self.eot_id = -1
        self.byte_fallback_start = -1
        self.trie = {}
        for i, piece in enumerate(vocab):
            if piece == b"<0x00>":
                self.byte_fallback_start = i
            elif piece in (b"<|eot_id|>", b"<|end|>", b"<|im_end|>"):      # src/tokenizer.cpp:22-24
                self.eot_id = i
            node = self.trie
            for c in piece:
                node = node.setdefault(c, {})
            if piece:
                node[-1] = i

    @classmethod
    def from_folder(cls, folder, vocab_size, bos_id, eos_id):
        path = os.path.join(folder, "tokenizer.json")
        if not os.path.exists(path):
            raise FileNotFoundError("no tokenizer.json in %s: give the prompt as token ids (--tokens)" % folder)
        with open(path) as f:
            tok = json.load(f)
        pieces = [""] * vocab_size
        for t, i in tok["model"]["vocab"].items():
            if i < vocab_size:
                pieces[i] = t
        for added in tok.get("added_tokens", []):
            if added["id"] < vocab_size:
                pieces[added["id"]] = added["content"]
        gpt2 = not tok["model"].get("byte_fallback", False)
        table = _gpt2_byte_alphabet()
        vocab = []
        for t in pieces:
            if gpt2:
                b = bytes(table.get(c, 0) for c in t)
            else:
                b = t.replace("▁", " ").encode("utf-8")
            vocab.append(b.replace(b"\0", b"\7"))
        return cls(vocab, bos_id, eos_id)

    def encode(self, text, bos=True):
        data = text.encode("utf-8") if isinstance(text, str) else bytes(text)
        out = [self.bos_id] if bos and self.bos_id is not None and self.bos_id >= 0 else []
        i, n = 0, len(data)
        while i < n:
            node, l, best, best_l = self.trie, 0, -1, 0
            while i + l < n:
                node = node.get(data[i + l])
                if node is None:
                    break
                l += 1
                if -1 in node:
                    best, best_l = node[-1], l
            if best < 0:
                if self.byte_fallback_start >= 0:
                    out.append(data[i] + self.byte_fallback_start)
                i += 1
            else:
                out.append(best)
                i += best_l
        return out

    def decode_one(self, prev_token, token):
        piece = self.vocab[token]
        if prev_token == self.bos_id and piece[:1] == b" ":
            return piece[1:]
        if self.byte_fallback_start >= 0 and 0 <= token - self.byte_fallback_start < 256:
            return bytes([token - self.byte_fallback_start])
        return piece
