"""SimpleTokenizer (mirror of tinygrad/llm/cli.py:11-74).  The reference's own tests need a vocabulary fetched from the network
(test/null/test_llm_tokenizer.py:7-33); what they hold offline is used here as it stands: the split pattern against the naive listing of every
code point (:51-58), the tekken from_gguf_kv vector (:84-98) and the stream-decoder vector (:100-108).  The merge order is pinned on a small
vocabulary worked by hand."""
import re, unicodedata
import pytest
from tinygrad_amd.tokenizer import SimpleTokenizer, _gpt2_byte_alphabet

def _enc(raw: bytes) -> str:
  inv = {b: ch for ch, b in _gpt2_byte_alphabet().items()}
  return "".join(inv[b] for b in raw)

def test_byte_alphabet_is_the_gpt2_table():
  tab = _gpt2_byte_alphabet()
  assert len(tab) == 256 and sorted(tab.values()) == list(range(256))
  assert tab["A"] == 0x41 and tab["Ġ"] == 0x20 and tab["Ċ"] == 0x0A and tab["Ā"] == 0x00 and tab["ÿ"] == 0xFF   # 'Ġ' = space, 'Ċ' = newline

def test_split_pattern_matches_naive_listing():
  # test/null/test_llm_tokenizer.py:51-58
  def naive(pre): return "".join(re.escape(chr(cp)) for cp in range(0x323b0) if unicodedata.category(chr(cp)).startswith(pre))
  ws, n, l = r"\t\n\x0b\x0c\r\x85" + naive("Z"), naive("N"), naive("L")
  naive_re = re.compile("(?i:'s|'t|'re|'ve|'m|'ll|'d)|" + f"[^\\r\\n{n}{l}]?[{l}]+|[{n}]{{1,3}}| ?[^{ws}{n}{l}]+[\\r\\n]*|[{ws}]*[\\r\\n]+|[{ws}]+(?![^{ws}])|[{ws}]+")
  sample = "hello world 한국어 中文 текст ١٢٣ 123 😊\n  \ttoday\n'équivalent ²³№ "
  tok = SimpleTokenizer({}, {})
  assert tok._split_to_word.findall(sample) == naive_re.findall(sample)
  assert len(tok._split_to_word.pattern) < 100_000
  assert len(tok._split_to_word.findall("The quick brown fox jumps over the lazy dog. " * 500)) == 5001

def test_merge_order_by_hand():
  """Vocabulary ids are merge ranks.  Word 'abcab': pairs ab (id 5), bc (id 4), ca (absent), ab -> bc has the lowest id and merges first:
  a|bc|a|b; then ab (5) vs 'abc' = a+bc (id 7) and bca (absent): ab wins: a|bc|ab; then a+bc = abc (7), bc+ab absent -> abc|ab; abc+ab absent: [7, 5]."""
  vocab = {"a": 0, "b": 1, "c": 2, "d": 3, "bc": 4, "ab": 5, "Ġ": 6, "abc": 7, "Ġd": 8, "dd": 9}     # 'Ġ' is the vocabulary's spelling of a space
  tok = SimpleTokenizer(vocab, {"<s>": 100, "<|end|>": 101}, eos_id=101)
  assert tok._encode_word(b"abcab") == [7, 5]
  assert tok._encode_word(b"abc") == [7]                        # a whole word in the vocabulary is looked up, not merged
  assert tok.encode("abc d") == [7, 8]                           # the pattern keeps the leading space with the letters
  assert tok.encode("<s>ab<|end|>dd") == [100, 5, 101, 9]
  assert tok.decode([100, 5, 101, 9, 8]) == "<s>ab<|end|>dd d"
  assert tok.is_end(101) and not tok.is_end(5)
  with pytest.raises(RuntimeError, match="token not found"): tok.encode("abz")
  with pytest.raises(ValueError): SimpleTokenizer({}, {}, preset="nope")
  assert SimpleTokenizer({}, {}, preset="qwen35").preset == "qwen2"

def test_leftmost_pair_wins_among_equal_ranks():
  tok = SimpleTokenizer({"a": 0, "aa": 1}, {})
  assert tok._encode_word(b"aaa") == [1, 0]                      # (aa)(a), not (a)(aa)

def test_bytes_outside_ascii_round_trip():
  raw = " \xec\x8b\xa4".encode()                                   # the same kind of input as the reference's test_llama_bytes (:45)
  vocab = {_enc(bytes([b])): 10 + i for i, b in enumerate(sorted(set(raw)))}
  tok = SimpleTokenizer(vocab, {})
  ids = tok.encode(" \xec\x8b\xa4")
  assert len(ids) == len(raw) and tok.decode(ids) == " \xec\x8b\xa4"

def test_from_gguf_kv_tekken_vector():
  # test/null/test_llm_tokenizer.py:84-98 (without the chat template, which is outside the built path)
  kv = {"tokenizer.ggml.tokens": ["<unk>", "<s>", "</s>", "[INST]", "[/INST]", "hello"], "tokenizer.ggml.token_type": [3, 3, 3, 3, 3, 1],
        "tokenizer.ggml.pre": "tekken", "tokenizer.ggml.eos_token_id": 2}
  tok = SimpleTokenizer.from_gguf_kv(kv)
  assert tok.encode("hello") == [5] and tok.encode("[INST]hello[/INST]") == [3, 5, 4]
  assert tok.eos_id == 2 and tok.bos_id is None and tok.eot_id is None and tok.preset == "tekken"

def test_stream_decoder_vector():
  # test/null/test_llm_tokenizer.py:100-108: token 25677 holds 3/4 of an emoji, token 138 completes it
  token_bytes = {25677: b"\x20\xf0\x9f\x98", 138: b"\x8a"}
  tok = SimpleTokenizer({_enc(v): k for k, v in token_bytes.items()}, {})
  dec = tok.stream_decoder()
  assert dec(25677) + dec(138) + dec() == " 😊"
