"""BPE tokenizer (host code behind the C ABI) against an independent implementation of the same published
algorithm: the `tokenizers` library's byte-level BPE built from the reference's own test assets
(source/test-suite/external/assets/gpt2_tokenizer/{tokens,merges}.txt, kept under tests/golden/), which is what
the reference's test compares with through tiktoken (test-tokenizer.lisp:26-37)."""
import json
import os

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ASSETS = os.path.join(HERE, "golden", "gpt2_tokenizer")

# the reference's three sentences (test-tokenizer.lisp:35-37) with the ids tiktoken's "gpt2" encoding gives
REFERENCE_SENTENCES = {
    "Say hello to me": [25515, 23748, 284, 502],
    "Hello world": [15496, 995],
    "What is the answer to the life, the world, and everything?":
        [2061, 318, 262, 3280, 284, 262, 1204, 11, 262, 995, 11, 290, 2279, 30],
}

SENTENCES = list(REFERENCE_SENTENCES) + [
    "", " ", "  ", "a", " a", "a ", "don't  stop   now\n\nIt's 2024!!  ", "we're they've I'm you'll he'd 'tis",
    "tabs\tand\r\nnewlines \n end ", "1234567890 3.14159 x86_64 foo_bar-baz", "naïve café — “quotes” … 日本語のテキスト ½ ²",
    "emoji 🙂🙃 mixed💥text", "     leading and trailing     ", "UPPER lower MiXeD 'S 'T", "\n", "a\n\n\nb", "!!!???...,,,",
]


@pytest.fixture(scope="module")
def assets():
    tokens = open(os.path.join(ASSETS, "tokens.txt"), encoding="utf-8").read()
    merges = open(os.path.join(ASSETS, "merges.txt"), encoding="utf-8").read()
    return tokens, merges


@pytest.fixture(scope="module")
def tok(assets):
    from caten_amd.tokenizer import make_bpe_tokenizer
    return make_bpe_tokenizer(*assets)


@pytest.fixture(scope="module")
def library_tok(assets, tmp_path_factory):
    transformers = pytest.importorskip("transformers")
    tokens, merges = assets
    d = tmp_path_factory.mktemp("gpt2tok")
    vocab = {s: i for i, s in enumerate(tokens.split(" ")[1:])}
    json.dump(vocab, open(d / "vocab.json", "w"))
    lines = [l.strip() for l in merges.split("\n")[1:] if l.strip()]
    open(d / "merges.txt", "w", encoding="utf-8").write("#version: 0.2\n" + "\n".join(lines) + "\n")
    return transformers.GPT2Tokenizer(str(d / "vocab.json"), str(d / "merges.txt"))


def test_vocabulary_size(tok):
    assert tok.vocab_size == 50257


@pytest.mark.parametrize("sentence,ids", REFERENCE_SENTENCES.items())
def test_reference_sentences(tok, sentence, ids):
    assert tok.encode(sentence) == ids
    assert tok.decode(ids) == sentence


@pytest.mark.parametrize("sentence", SENTENCES)
def test_encode_decode_match_library(tok, library_tok, sentence):
    want = library_tok.encode(sentence)
    assert tok.encode(sentence) == want
    assert tok.decode(want) == sentence  # byte-level BPE round-trips any text


def test_every_token_decodes_to_its_bytes(tok, library_tok):
    ids = list(range(0, 50257, 97)) + [198, 220, 50256]
    for i in ids:
        assert tok.decode([i]) == library_tok.decode([i], clean_up_tokenization_spaces=False)


def test_unknown_symbol_and_bad_id():
    from caten_amd import HipError
    from caten_amd.tokenizer import make_bpe_tokenizer
    t = make_bpe_tokenizer(" a b ab", "\na b")  # ids: a=0 b=1 ab=2; rank 0 merges a+b
    assert t.encode("ab") == [2]
    assert t.encode("ba") == [1, 0]
    assert t.encode("abc") == [2, 0]  # 'c' is not in the vocabulary: id 0, as the reference's (or ... 0)
    assert t.decode([2, 1]) == "abb"
    with pytest.raises(HipError):
        t.decode([3])
    with pytest.raises(TypeError):
        t.encode(b"bytes")


def _small_vocab(assets, n=1000):
    """The first n symbols of the GPT-2 vocabulary (256 byte symbols + the first n-256 merges, which is how that
    vocabulary is numbered) and exactly those merges: a consistent tokenizer for a model with n embeddings."""
    tokens, merges = assets
    toks = tokens.split(" ")[1:n + 1]
    lines = merges.split("\n")[1:n - 256 + 1]
    return " " + " ".join(toks), "\n" + "\n".join(lines)


def test_small_vocabulary_is_consistent(assets):
    from caten_amd.tokenizer import make_bpe_tokenizer
    t = make_bpe_tokenizer(*_small_vocab(assets))
    assert t.vocab_size == 1000
    text = "The quick brown fox jumps over the lazy dog, 42 times!"
    ids = t.encode(text)
    assert max(ids) < 1000 and len(ids) < len(text)  # merges happen, nothing falls outside the vocabulary
    assert t.decode(ids) == text


def test_tokenizer_from_gguf_metadata(tmp_path, assets):
    from caten_amd.gguf import GGUF, write_gguf
    from caten_amd.tokenizer import gguf_bpe_tokenizer, make_bpe_tokenizer
    import numpy as np
    toks, merges = _small_vocab(assets, 400)
    path = str(tmp_path / "tok.gguf")
    write_gguf(path, {"general.architecture": "gpt2", "tokenizer.ggml.tokens": toks.split(" ")[1:],
                      "tokenizer.ggml.merges": merges.split("\n")[1:]},
               [("dummy.weight", "f32", (2, 2), np.zeros((2, 2), np.float32))])
    g = GGUF(path)
    a, b = gguf_bpe_tokenizer(g), make_bpe_tokenizer(toks, merges)
    for text in ("hello there", "in the end", "a b  c"):
        assert a.encode(text) == b.encode(text)
    g.close()
    with pytest.raises(KeyError):
        path2 = str(tmp_path / "notok.gguf")
        write_gguf(path2, {"general.architecture": "gpt2"}, [("dummy.weight", "f32", (2, 2), np.zeros((2, 2), np.float32))])
        gguf_bpe_tokenizer(GGUF(path2))


@pytest.mark.gpu
def test_generate_text_end_to_end(assets):
    """String in, string out through the decoder session (gpt2-generate): the text is the decoding of the prompt
    ids followed by the ids the id-level loop yields."""
    from caten_amd import synth, llm
    from caten_amd.tokenizer import make_bpe_tokenizer
    t = make_bpe_tokenizer(*_small_vocab(assets, 1000))
    cfg = synth.GPT2_CONFIGS["gpt2-tiny"]  # vocabulary of 1000
    model = llm.make_gpt2(cfg, llm.gpt2_state_dict(synth.gpt2_weights(cfg, seed=0), "q8_0"))
    text = "Say hello to me"
    out = llm.gpt2_generate_text(model, t, text, max_length=12)
    prompt = t.encode(text)
    want = t.decode(prompt + llm.gpt2_generate(model, prompt, 12, on_device=False))
    assert out == want and out.startswith(text)
    with pytest.raises(AssertionError):
        llm.gpt2_generate_text(model, t, text, max_length=3, expected="something else")
    model.close()
