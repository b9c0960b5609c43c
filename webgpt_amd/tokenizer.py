"""Tokenizers of the reference (tokenizer.js): a character-level table and GPT-2 byte-pair
encoding. The BPE vocabulary is rebuilt from the merges file alone when `gpt_tokens.json` is
not at hand: ids 0..255 are the byte symbols in `bytes_to_unicode` order, id 256 + r is the
concatenation of merge r, and the last id is <|endoftext|> (how GPT-2's encoder.json was made)."""
import json

import regex


class Tokenizer:
    """tokenizer.js:1-23."""

    def __init__(self):
        self.encoder = None
        self.decoder = None
        self.vocab_size = None

    def load(self, *args, **kwargs):
        raise NotImplementedError("Not implemented.")

    def getVocabSize(self):
        return self.vocab_size

    def encode(self, text):
        raise NotImplementedError("Not implemented.")

    def decode(self, arr):
        raise NotImplementedError("Not implemented.")


class SimpleTokenizer(Tokenizer):
    """tokenizer.js:25-45: one id per character, from a {character: id} JSON."""

    def load(self, path=None, chars=None):
        if chars is not None:                      # nanoGPT's char-level table: sorted(set(text))
            self.encoder = {c: i for i, c in enumerate(sorted(set(chars)))}
        else:
            with open(path, encoding="utf-8") as f:
                self.encoder = json.load(f)
        self.decoder = {v: k for k, v in self.encoder.items()}
        self.vocab_size = len(self.encoder)
        return self

    def encode(self, text):
        return [self.encoder[c] for c in text]

    def decode(self, arr):
        return "".join(self.decoder[int(x)] for x in arr)


def bytes_to_unicode():
    """tokenizer.js:177-194: byte -> printable character; printable bytes map to themselves,
    the other 68 to U+0100 onwards in ascending byte order."""
    bs = list(range(ord("!"), ord("~") + 1)) + list(range(ord("¡"), ord("¬") + 1)) + list(range(ord("®"), ord("ÿ") + 1))
    cs = bs[:]
    n = 0
    for b in range(256):
        if b not in bs:
            bs.append(b)
            cs.append(256 + n)
            n += 1
    return {b: chr(c) for b, c in zip(bs, cs)}


def get_pairs(word):
    return {(a, b) for a, b in zip(word[:-1], word[1:])}


class GPT2Tokenizer(Tokenizer):
    """tokenizer.js:50-160 (a port of GPT-3-Encoder)."""

    PAT = regex.compile(r"'s|'t|'re|'ve|'m|'ll|'d| ?\p{L}+| ?\p{N}+| ?[^\s\p{L}\p{N}]+|\s+(?!\S)|\s+")

    def load(self, bpe_path, tokens_path=None):
        with open(bpe_path, encoding="utf-8") as f:
            lines = f.read().split("\n")
        # first line is the version header, the last element the empty string after the final newline
        merges = [tuple(x.split()) for x in lines[1:] if x.strip()]
        self.byte_encoder = bytes_to_unicode()
        self.byte_decoder = {v: k for k, v in self.byte_encoder.items()}
        if tokens_path is not None:
            with open(tokens_path, encoding="utf-8") as f:
                self.encoder = json.load(f)
        else:
            symbols = list(self.byte_encoder.values()) + [a + b for a, b in merges] + ["<|endoftext|>"]
            self.encoder = {s: i for i, s in enumerate(symbols)}
        self.decoder = {v: k for k, v in self.encoder.items()}
        self.bpe_ranks = {m: i for i, m in enumerate(merges)}
        self.cache = {}
        self.vocab_size = len(self.encoder)
        return self

    def bpe(self, token):
        if token in self.cache:
            return self.cache[token]
        word = list(token)
        pairs = get_pairs(word)
        if not pairs:
            return token
        while True:
            bigram = min(pairs, key=lambda p: self.bpe_ranks.get(p, 10e10))
            if bigram not in self.bpe_ranks:
                break
            first, second = bigram
            new_word = []
            i = 0
            while i < len(word):
                try:
                    j = word.index(first, i)
                except ValueError:
                    new_word.extend(word[i:])
                    break
                new_word.extend(word[i:j])
                i = j
                if word[i] == first and i < len(word) - 1 and word[i + 1] == second:
                    new_word.append(first + second)
                    i += 2
                else:
                    new_word.append(word[i])
                    i += 1
            word = new_word
            if len(word) == 1:
                break
            pairs = get_pairs(word)
        out = " ".join(word)
        self.cache[token] = out
        return out

    def encode(self, text):
        if getattr(self, "byte_encoder", None) is None:
            raise RuntimeError("Tokenizer not loaded.")
        ids = []
        for token in self.PAT.findall(text):
            token = "".join(self.byte_encoder[b] for b in token.encode("utf-8"))
            ids.extend(self.encoder[x] for x in self.bpe(token).split(" "))
        return ids

    def decode(self, tokens):
        if getattr(self, "byte_decoder", None) is None:
            raise RuntimeError("Tokenizer not loaded.")
        text = "".join(self.decoder[int(x)] for x in tokens)
        return bytes(self.byte_decoder[c] for c in text).decode("utf-8", errors="replace")
