"""GPT-2 byte-level BPE tokenizer (host side): the reference's checks (tests_tokenizer.rs: vocabulary size, encode /
decode round trips over English, punctuation, numbers, CJK, emoji, whitespace, code, empty and single-character
texts, <|endoftext|> alone and inside text) on a small vocabulary trained here, since no vocabulary file is in the
image; the merge algorithm and the split pattern are checked against the `tokenizers` library's byte-level BPE on the
same vocabulary, and against splits GPT-2's pattern is known to make.  Token ids of the real r50k_base table run only
where AGPU_GPT2_VOCAB names it: parity on the real vocabulary is otherwise unpinned.
"""
import collections
import json
import os
import random

import pytest

import __graft_entry__ as entry

entry.load_package()
from async_gpu_amd import tokenizer as T  # noqa: E402

CORPUS = """The quick brown fox jumps over the lazy dog. The capital of France is Paris, and the capital of Japan is Tokyo.
In a world where AI writes code, fn main() { println!("hello"); } is what it's all about; isn't it? They've said we'll see.
Wait... really?! Yes! 100% sure. 123 + 456 = 579, and 3.14 * 2 = 6.28.   Tabs\there\nand\nnewlines  plus   spaces.
Hello 你好世界, I love Rust \U0001f980\U0001f680 and café naïve über straße. aaaaaaaaaaaaaaaa bbbb aaaa the the the then there.
"""

TEXTS = [
    "Hello, world!",
    "The quick brown fox jumps over the lazy dog. 123 + 456 = 579",
    "Wait... really?! Yes! 100% sure.",
    "123 + 456 = 579, and 3.14 * 2 = 6.28",
    "Hello 你好世界",
    "I love Rust \U0001f980\U0001f680",
    "tabs\there\nand\nnewlines  plus   spaces",
    "fn main() { println!(\"hello\"); }",
    "",
    "A",
    "aaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaaa",
    "Pneumonoultramicroscopicsilicovolcanoconiosis",
    "it's they've we'll I'm he'd don't you're",
    "  leading and trailing  ",
    "\n\n\nline\r\nbreaks\n",
    "mixed nbsp emspace",
]


def train(corpus, n_merges):
    """Plain byte-pair training: the most frequent adjacent pair first, ties by the pair's bytes."""
    split = T.regex.compile(T._PATTERN)
    words = collections.Counter(tuple(bytes([b]) for b in w.encode("utf-8")) for w in split.findall(corpus))
    merges = []
    for _ in range(n_merges):
        pairs = collections.Counter()
        for w, c in words.items():
            for a, b in zip(w, w[1:]):
                pairs[(a, b)] += c
        if not pairs:
            break
        (a, b), _ = min(pairs.items(), key=lambda kv: (-kv[1], kv[0]))
        merges.append((a, b))
        new = collections.Counter()
        for w, c in words.items():
            out, i = [], 0
            while i < len(w):
                if i + 1 < len(w) and w[i] == a and w[i + 1] == b:
                    out.append(a + b)
                    i += 2
                else:
                    out.append(w[i])
                    i += 1
            new[tuple(out)] += c
        words = new
    b2u = T.bytes_to_unicode()
    ranks = {bytes([b]): i for i, b in enumerate(b2u)}  # the first 256 ids in GPT-2's byte order
    for a, b in merges:
        ranks.setdefault(a + b, len(ranks))
    return ranks, merges


@pytest.fixture(scope="module")
def small():
    ranks, merges = train(CORPUS, 400)
    return T.Gpt2Tokenizer(ranks), ranks, merges


def test_vocab_size_and_special_token(small):
    tok, ranks, _ = small
    assert tok.vocab_size() == len(ranks) + 1
    assert tok.encode(T.ENDOFTEXT) == [len(ranks)]
    assert tok.encode("") == []
    ids = tok.encode("Hello" + T.ENDOFTEXT + "world")
    assert ids.count(len(ranks)) == 1 and tok.decode(ids) == "Hello" + T.ENDOFTEXT + "world"
    assert ids == tok.encode("Hello") + [len(ranks)] + tok.encode("world")
    assert T.GPT2_VOCAB_SIZE == 50257 and T.ENDOFTEXT_TOKEN_ID == 50256


@pytest.mark.parametrize("text", TEXTS)
def test_round_trip(small, text):
    tok = small[0]
    ids = tok.encode(text)
    assert (len(ids) > 0) == (len(text) > 0)
    assert all(0 <= i < tok.vocab_size() for i in ids)
    assert tok.decode(ids) == text


def test_merges_shorten(small):
    tok = small[0]
    # words of the training text have become few tokens, unseen bytes stay bytes
    assert len(tok.encode(" the")) == 1 and len(tok.encode(" capital")) <= 3
    assert len(tok.encode("Ж")) == 2  # two UTF-8 bytes never seen together


def test_split_pattern_known_cases():
    split = T.regex.compile(T._PATTERN).findall
    assert split("Hello world") == ["Hello", " world"]
    assert split("it's") == ["it", "'s"]
    assert split("we'll they've I'm") == ["we", "'ll", " they", "'ve", " I", "'m"]
    assert split("a  b") == ["a", " ", " b"]          # the run of blanks gives up its last one to the word
    assert split("x\n\ny") == ["x", "\n", "\n", "y"]  # likewise: the last line break stands alone before a word
    assert split("x\n\n") == ["x", "\n\n"]
    assert split("abc123") == ["abc", "123"]
    assert split("a !?b") == ["a", " !?", "b"]
    assert split("end  ") == ["end", "  "]
    assert split("你好 42") == ["你好", " 42"]


def test_against_the_tokenizers_library(small):
    tokenizers = pytest.importorskip("tokenizers")
    tok, ranks, merges = small
    b2u = T.bytes_to_unicode()
    as_text = lambda bs: "".join(b2u[b] for b in bs)
    hf = tokenizers.Tokenizer(tokenizers.models.BPE(vocab={as_text(t): i for t, i in ranks.items()},
                                                    merges=[(as_text(a), as_text(b)) for a, b in merges]))
    hf.pre_tokenizer = tokenizers.pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=True)
    hf.decoder = tokenizers.decoders.ByteLevel()
    hf.add_special_tokens([T.ENDOFTEXT])
    rng = random.Random(7)
    alphabet = list("abcdefghijklmnopqrstuvwxyzTHE .,!?'\n\t0123456789") + ["你", "é", "\U0001f980", " the", " of", "'s", "  "]
    texts = TEXTS + CORPUS.split("\n") + ["".join(rng.choice(alphabet) for _ in range(rng.randrange(1, 80))) for _ in range(300)]
    texts.append("Hello" + T.ENDOFTEXT + "world")
    for text in texts:
        assert tok.encode(text) == hf.encode(text).ids, text
        ids = tok.encode(text)
        assert tok.decode(ids) == hf.decode(ids, skip_special_tokens=False) == text


def test_vocabulary_files(small, tmp_path):
    tok, ranks, merges = small
    p = tmp_path / "small.tiktoken"
    tok.save_tiktoken_file(str(p))
    again = T.Gpt2Tokenizer.from_tiktoken_file(str(p))
    b2u = T.bytes_to_unicode()
    as_text = lambda bs: "".join(b2u[b] for b in bs)
    vocab = {as_text(t): i for t, i in ranks.items()}
    vocab[T.ENDOFTEXT] = len(ranks)
    (tmp_path / "g").mkdir()
    (tmp_path / "g" / "encoder.json").write_text(json.dumps(vocab), encoding="utf-8")
    (tmp_path / "g" / "vocab.bpe").write_text("#version: 0.2\n" + "\n".join(f"{as_text(a)} {as_text(b)}" for a, b in merges) + "\n",
                                              encoding="utf-8")
    from_dir = T.Gpt2Tokenizer.new(str(tmp_path / "g"))
    for text in TEXTS + ["x" + T.ENDOFTEXT]:
        assert again.encode(text) == tok.encode(text) == from_dir.encode(text)
    assert from_dir.vocab_size() == tok.vocab_size()
    (tmp_path / "g" / "vocab.bpe").write_text("q q\n", encoding="utf-8")  # a merge whose result is no token
    with pytest.raises(T.TokenizerError) as e:
        T.Gpt2Tokenizer.new(str(tmp_path / "g"))
    assert e.value.kind == "init"


def test_errors(small, monkeypatch):
    tok, ranks, _ = small
    with pytest.raises(T.TokenizerError) as e:
        tok.decode([10 ** 6])
    assert e.value.kind == "decode"
    with pytest.raises(T.TokenizerError) as e:
        tok.decode(tok.encode("é")[:1] if len(tok.encode("é")) > 1 else [ranks[b"\xc3"]])  # half a character
    assert e.value.kind == "decode"
    assert tok.decode_bytes([ranks[b"\xc3"]]) == b"\xc3"
    monkeypatch.delenv("AGPU_GPT2_VOCAB", raising=False)
    with pytest.raises(T.TokenizerError) as e:
        T.Gpt2Tokenizer.new()
    assert e.value.kind == "init"
    with pytest.raises(T.TokenizerError):
        T.Gpt2Tokenizer({b"a": 0})  # not byte-level


@pytest.mark.skipif(not os.environ.get("AGPU_GPT2_VOCAB"), reason="the r50k_base table is not in the image; set AGPU_GPT2_VOCAB")
def test_real_vocabulary():
    tok = T.Gpt2Tokenizer.new()
    assert tok.vocab_size() == T.GPT2_VOCAB_SIZE
    assert tok.encode(T.ENDOFTEXT) == [T.ENDOFTEXT_TOKEN_ID]
    assert tok.encode("Hello, world!") == [15496, 11, 995, 0]
    for text in TEXTS:
        assert tok.decode(tok.encode(text)) == text
