"""Tokenizers (tokenizer.js:25-160). The fixture tests/golden/vocab_head1000.bpe is the header
and the first 1000 merges of GPT-2's public vocab.bpe (data the reference ships under
weights/tokenization); ids below 1256 do not depend on the rest of the file. Known answers are
GPT-2's published vocabulary: byte symbols first ("!" = 0, "A" = 32, "\\n" = 198, " " = 220),
then one id per merge in file order (" t" = 256, " a" = 257, "he" = 258, "in" = 259, " the" = 262)."""
import json
import os
import shutil
import subprocess

import pytest

from webgpt_amd.tokenizer import GPT2Tokenizer, SimpleTokenizer, bytes_to_unicode

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BPE = os.path.join(ROOT, "tests", "golden", "vocab_head1000.bpe")
NODE = shutil.which("node")
TEXTS = ["!", "A", "\n", " ", " t", " a", "he", "in", " the", " the and in", "Hello", "it's 42 days...  \n\n x", "Héllo wörld ☃"]


def test_byte_table():
    m = bytes_to_unicode()
    assert len(m) == 256 and len(set(m.values())) == 256
    assert m[ord("!")] == "!" and m[ord("~")] == "~" and m[0] == "Ā" and m[32] == "Ġ" and m[10] == "Ċ"
    order = list(m.values())
    assert order.index("!") == 0 and order.index("A") == 32 and order.index("Ċ") == 198 and order.index("Ġ") == 220


def test_gpt2_known_ids_and_round_trip():
    t = GPT2Tokenizer().load(BPE)
    assert t.getVocabSize() == 256 + 1000 + 1 and t.encoder["<|endoftext|>"] == 1256
    want = {"!": [0], "A": [32], "\n": [198], " ": [220], " t": [256], " a": [257], "he": [258], "in": [259], " the": [262],
            " the and in": [262, 290, 287]}
    for text, ids in want.items():
        assert t.encode(text) == ids, text
    for text in TEXTS:
        assert t.decode(t.encode(text)) == text
    # the pre-tokenizer keeps a run of spaces apart from the space that leads the next word
    assert t.decode(t.encode("a  b")[1:2]) == " "
    with pytest.raises(RuntimeError, match="Tokenizer not loaded."):
        GPT2Tokenizer().encode("x")


def test_simple_tokenizer(tmp_path):
    s = SimpleTokenizer().load(chars="hello world")
    assert s.getVocabSize() == 8 and s.encode("low") == [4, 5, 7] and s.decode([3, 2, 2]) == "hee"
    p = tmp_path / "simple_tokens.json"
    p.write_text(json.dumps({"a": 0, "b": 1, "\n": 2}))
    f = SimpleTokenizer().load(str(p))
    assert f.encode("ab\nba") == [0, 1, 2, 1, 0] and f.decode([2, 0]) == "\na"


@pytest.mark.skipif(NODE is None, reason="node is not installed")
def test_js_tokenizers_agree_with_python():
    r = subprocess.run([NODE, os.path.join(ROOT, "tests", "js", "tokenizer_checks.js"), BPE, *TEXTS],
                       capture_output=True, text=True, timeout=120, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    out = json.loads(r.stdout.strip().splitlines()[-1])
    t = GPT2Tokenizer().load(BPE)
    assert out["vocab_size"] == t.getVocabSize() and out["eot"] == 1256
    assert out["ids"] == [t.encode(x) for x in TEXTS]
    assert out["round"] == TEXTS
    assert out["simple"] == {"ids": [4, 5, 7], "text": "hee", "n": 8}


FULL_BPE = "/root/reference/weights/tokenization/vocab.bpe"
# GPT-2's published encodings (the ids every GPT-2 tokenizer gives for these strings); they need merges far beyond
# the first 1000, so they run only where the reference's complete merges file is readable
PUBLISHED = {"Hello world": [15496, 995], " Hello": [18435],
             "The quick brown fox jumps over the lazy dog.": [464, 2068, 7586, 21831, 18045, 625, 262, 16931, 3290, 13]}


@pytest.mark.skipif(not os.access(FULL_BPE, os.R_OK), reason="the reference's complete vocab.bpe is not on this machine")
def test_gpt2_published_ids_with_the_complete_merges_file():
    t = GPT2Tokenizer().load(FULL_BPE)
    assert t.getVocabSize() == 50257 and t.encoder["<|endoftext|>"] == 50256
    for text, ids in PUBLISHED.items():
        assert t.encode(text) == ids and t.decode(ids) == text, text
    if NODE is not None:
        r = subprocess.run([NODE, os.path.join(ROOT, "tests", "js", "tokenizer_checks.js"), FULL_BPE, *PUBLISHED],
                           capture_output=True, text=True, timeout=120, cwd=ROOT)
        assert r.returncode == 0, r.stderr[-2000:]
        out = json.loads(r.stdout.strip().splitlines()[-1])
        assert out["vocab_size"] == 50257 and out["eot"] == 50256
        assert out["ids"] == list(PUBLISHED.values()) and out["round"] == list(PUBLISHED)


@pytest.mark.gpu
def test_generate_from_text(device):
    """generate(prompt: string) end to end (model.js:53-102) with the character tokenizer."""
    import numpy as np
    from oracle import ref
    from webgpt_amd import synth
    from webgpt_amd.model import GPT
    from helpers import make_model, oracle_weights, small_cfg
    tok = SimpleTokenizer().load(chars="abcdefghijklmnopqrstuvwxyz .,\n")
    cfg = small_cfg(n_layer=2, n_head=2, n_embd=128, n_ctx=32, vocab_size=32)
    tensors = make_model(cfg, 6)
    gpt = GPT(None, "char", tensors=tensors, params=synth.model_params(cfg), tokenizer=tok)
    gpt.initialize()
    try:
        text = "".join(gpt.generate("hello world", 6, 1, 1.0))
        hist = tok.encode("hello world")
        p, w = synth.model_params(cfg), oracle_weights(tensors, cfg)
        want = []
        for _ in range(6):
            nxt = int(np.argmax(ref.forward(p, w, np.array(hist, np.int32))))
            want.append(nxt)
            hist.append(nxt)
        assert text == tok.decode(want)
    finally:
        gpt.unloadBuffers()
