"""The byte-level BPE read from tokenizer.json (vectors of src/qwen.rs:359-453 of the reference) and the
command line's argument rules (qwen-infer/src/main.rs:76-148).  The reference's 314 real cases
(tests/fixtures/qwen_cases.jsonl) need the real tokenizer.json, which is not available: parity unpinned."""
import json

import pytest

from tokenizer_amd.cli import ArgError, parse_args
from tokenizer_amd.tokenizer import Tokenizer, TokenizerError, UnknownToken, bytes_to_unicode_reverse


def tiny_file(pattern="[\\s\\S]+"):
    reverse = bytes_to_unicode_reverse()
    of_byte = {byte: ch for ch, byte in reverse.items()}
    vocab = {of_byte[b]: b for b in range(256)}
    vocab["ab"] = 256            # the merge result has id 256, not the merge's rank 0
    return {"added_tokens": [{"id": 300, "content": "<|endoftext|>", "normalized": False, "special": True}],
            "normalizer": {"type": "NFC"},
            "pre_tokenizer": {"type": "Sequence", "pretokenizers": [
                {"type": "Split", "pattern": {"Regex": pattern}, "behavior": "Isolated", "invert": False},
                {"type": "ByteLevel", "add_prefix_space": False, "use_regex": False}]},
            "model": {"type": "BPE", "vocab": vocab, "merges": ["a b"]}}


def test_bytes_to_unicode_maps_the_known_bytes():
    reverse = bytes_to_unicode_reverse()
    assert len(reverse) == 256 and len(set(reverse.values())) == 256
    assert reverse["Ā"] == 0 and reverse["Ġ"] == ord(" ")
    assert reverse["!"] == ord("!") and reverse["a"] == ord("a")


def test_merges_by_rank_not_id_and_applies_nfc(tmp_path):
    path = tmp_path / "tokenizer.json"
    path.write_text(json.dumps(tiny_file()))
    tok = Tokenizer.load_qwen(str(path))
    assert tok.encode("ab") == [256]
    assert tok.encode("ba") == [ord("b"), ord("a")]
    assert tok.encode("aba") == [256, ord("a")]
    assert tok.decode([256]) == "ab"
    composed = tok.encode("é")
    assert tok.encode("é") == composed and composed != [ord("e"), 0xCC, 0x81]
    assert tok.decode(composed) == "é"
    ids = tok.encode("a<|endoftext|>b")
    assert ids == [ord("a"), 300, ord("b")] and tok.decode(ids) == "a<|endoftext|>b"
    with pytest.raises(UnknownToken):
        tok.decode([257])
    assert tok.decode_bytes([0xC3]) == b"\xc3"       # bytes, not replaced characters


def test_gaps_the_pattern_leaves_are_pieces_too():
    tok = Tokenizer.from_json(tiny_file(pattern="a+"))
    assert tok.encode("xaabx") == [ord("x"), ord("a"), ord("a"), ord("b"), ord("x")]
    tok = Tokenizer.from_json(tiny_file(pattern="(?i:'s)|[^\\r\\n\\p{L}\\p{N}]?\\p{L}+|\\p{N}| ?[^\\s\\p{L}\\p{N}]+[\\r\\n]*|\\s*[\\r\\n]+|\\s+(?!\\S)|\\s+"))
    assert tok.decode(tok.encode("ab  cab 12's")) == "ab  cab 12's"
    assert tok.encode("ab ab")[:1] == [256]


def test_added_tokens_are_found_leftmost_first_and_the_longest_of_those_that_start_together():
    # src/rank.rs:368-447
    data = tiny_file()
    data["added_tokens"] += [{"id": 301, "content": "<|end", "normalized": False},
                             {"id": 302, "content": "<|endoftext|>x", "normalized": False}]
    tok = Tokenizer.from_json(data)
    assert tok.encode("a<|endoftext|>xb<|endq") == [ord("a"), 302, ord("b"), 301, ord("q")]
    assert tok.encode("<|endoftext|>") == [300] and tok.encode("") == []
    assert tok.decode(tok.encode("ab<|end<|endoftext|>")) == "ab<|end<|endoftext|>"
    assert tok.vocab_size() == 303


@pytest.mark.parametrize("change, word", [
    (lambda f: f["added_tokens"].append(dict(f["added_tokens"][0], id=301)), "listed twice"),
    (lambda f: f["added_tokens"][0].update(id=97), "token id 97 is given to"),
    (lambda f: f["model"]["vocab"].update({"\u00ad": 400}), "spells no byte"),
    (lambda f: f["model"].update(merges=["a b", "a b"]), "produce the same bytes"),
    (lambda f: f["pre_tokenizer"]["pretokenizers"].pop(1), "no ByteLevel step"),
    (lambda f: f["added_tokens"][0].update(normalized=True), "normalized"),
    (lambda f: f.update(normalizer={"type": "NFKC"}), "NFC"),
    (lambda f: f.update(normalizer=None), "no normalizer"),
    (lambda f: f["pre_tokenizer"]["pretokenizers"][0].update(behavior="Removed"), "Isolated"),
    (lambda f: f["pre_tokenizer"]["pretokenizers"][1].update(use_regex=True), "use_regex"),
    (lambda f: f["model"].update(type="Unigram"), "BPE"),
    (lambda f: f["model"]["vocab"].pop("a"), "missing single-byte token 97"),
    (lambda f: f["model"].update(merges=["a c", "a c"]), "not in the vocab"),
    (lambda f: f["model"].update(merges=["ab"]), "no space"),
])
def test_files_of_another_kind_are_refused(change, word):
    data = tiny_file()
    change(data)
    with pytest.raises(TokenizerError) as err:
        Tokenizer.from_json(data)
    assert word in str(err.value)


def test_command_line_arguments():
    args = parse_args(["--model", "m", "The capital of France is"])
    assert (args["max_tokens"], args["temperature"], args["top_p"], args["seed"], args["stop"]) == (20, 0.0, 1.0, 0, [])
    args = parse_args(["--max-tokens", "7", "--temperature", "0.5", "--top-p", "0.9", "--seed", "3",
                       "--stop", "a", "--stop", "b", "--model", "m", "hi"])
    assert (args["max_tokens"], args["temperature"], args["top_p"], args["seed"], args["stop"], args["prompt"]) == \
        (7, 0.5, 0.9, 3, ["a", "b"], "hi")
    for bad, word in ((["-x", "p"], "unknown argument -x"), (["a", "b"], "only one prompt"),
                      (["--max-tokens"], "needs a value"), (["--max-tokens", "x", "p"], "--max-tokens x"),
                      (["--seed", "1.5", "p"], "--seed wants an integer")):
        with pytest.raises(ArgError) as err:
            parse_args(bad)
        assert word in str(err.value)


def test_generate_takes_text_with_a_tokenizer(model_folders):
    """`generate(model, text, params, tokenizer=...)`: the text is encoded, the sampled ids are decoded."""
    from cpu_engine import cpu_engine
    from tokenizer_amd.engine import GenerateParams, generate
    tok = Tokenizer.from_json(tiny_file())
    engine = cpu_engine(model_folders["A"])                     # vocabulary 256: every byte is a token
    from_text = generate(engine, "bbaa!", GenerateParams.greedy(5), tokenizer=tok)
    from_ids = generate(cpu_engine(model_folders["A"]), tok.encode("bbaa!"), GenerateParams.greedy(5))
    assert from_text.tokens == from_ids.tokens and len(from_text.tokens) == 5
    assert from_text.text == tok.decode_bytes(from_text.tokens).decode("utf-8", errors="replace")
    with pytest.raises(ValueError):
        generate(engine, "abba", GenerateParams.greedy(1))


def test_merges_in_the_host_library_follow_the_rule_spelled_out_here():
    """Random vocabularies over a small alphabet: the ids the tokenizer gives (its merge loop runs in the C++ host
    library) against the rule written out plainly: join the neighbouring pair whose joined bytes have the lowest
    rank, the leftmost of equals, until no pair has a rank (src/rank.rs:536-586)."""
    import random
    reverse = bytes_to_unicode_reverse()
    of_byte = {byte: ch for ch, byte in reverse.items()}
    spell = lambda raw: "".join(of_byte[b] for b in raw)

    def plainly(piece, ranks, ids):
        parts = [piece[i:i + 1] for i in range(len(piece))]
        while True:
            ranked = [(ranks[a + b], i) for i, (a, b) in enumerate(zip(parts, parts[1:])) if a + b in ranks]
            if not ranked:
                return [ids[p] for p in parts]
            _, at = min(ranked)
            parts[at:at + 2] = [parts[at] + parts[at + 1]]

    for seed in range(8):
        rng = random.Random(seed)
        ids = {bytes([b]): b for b in range(256)}
        merges, ranks = [], {}
        tokens = [b"a", b"b", b"c", b" "]
        for _ in range(rng.randint(3, 40)):
            left, right = rng.choice(tokens), rng.choice(tokens)
            if left + right in ranks or len(left + right) > 6:
                continue
            ranks[left + right] = len(merges)
            ids[left + right] = 256 + len(merges)
            merges.append(f"{spell(left)} {spell(right)}")
            tokens.append(left + right)
        data = tiny_file(pattern=" ?[abc]+| +")
        data["model"]["vocab"] = {spell(raw): token for raw, token in ids.items()}
        data["model"]["merges"] = merges
        tok = Tokenizer.from_json(data)
        for _ in range(30):
            text = "".join(rng.choice("abc ") for _ in range(rng.randint(1, 40)))
            want = []
            for piece in tok.pattern.findall(text):
                want += plainly(piece.encode(), ranks, ids)
            assert tok.encode(text) == want, (seed, text)
            assert tok.decode(want) == text
    long_piece = "ab" * 400                                    # more parts than the first buffer holds
    assert tok.decode(tok.encode(long_piece)) == long_piece


def test_the_tokenizer_is_chosen_by_what_the_file_declares(tmp_path):
    from tokenizer_amd.tokenizer import load_tokenizer, register_tokenizer, registered_tokenizers
    folder = tmp_path / "model"
    folder.mkdir()
    (folder / "tokenizer.json").write_text(json.dumps(tiny_file()))
    tok = load_tokenizer(str(folder))                                  # a folder, or the file itself
    assert isinstance(tok, Tokenizer) and tok.encode("ab") == [256]
    assert Tokenizer.load(str(folder / "tokenizer.json")).encode("ab") == [256]
    # A file of another kind is refused with what it declares and what is known ...
    other = {"model": {"type": "WordLevel", "vocab": {"a": 0, "b": 1}}, "pre_tokenizer": {"type": "Whitespace"}}
    (folder / "tokenizer.json").write_text(json.dumps(other))
    with pytest.raises(TokenizerError, match="model type 'WordLevel'.*byte_level_bpe"):
        load_tokenizer(str(folder))
    # ... until a kind that reads it is registered, from outside the package.

    class Words:
        def __init__(self, data):
            self.ids = data["model"]["vocab"]

        def encode(self, text):
            return [self.ids[word] for word in text.split()]

    if "toy_words" not in registered_tokenizers():
        register_tokenizer("toy_words", lambda data: data.get("model", {}).get("type") == "WordLevel", Words)
    assert load_tokenizer(str(folder)).encode("b a b") == [1, 0, 1]
    with pytest.raises(ValueError, match="already registered"):
        register_tokenizer("toy_words", lambda data: False, Words)
    with pytest.raises(TokenizerError, match="cannot read"):
        load_tokenizer(str(tmp_path / "nowhere"))
