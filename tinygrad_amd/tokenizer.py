"""Byte-level BPE tokenizer over the vocabulary a GGUF file carries: the mirror of SimpleTokenizer (tinygrad/llm/cli.py:11-74), so that text
goes in and comes out of Transformer.generate without any other package.  Host-only Python, as in the reference.

Text is cut at special tokens first, each remaining stretch into words by the llama-3 pre-tokenizer pattern (llama.cpp's LLAMA_VOCAB_PRE_TYPE_LLAMA3
regex with \\p{L} / \\p{N} / whitespace spelled out as code point ranges), and every word is encoded from its UTF-8 bytes: a word that is a
vocabulary entry is that token; otherwise adjacent pieces are merged, always the pair whose merged form has the lowest token id first, until
no adjacent pair is in the vocabulary (ids double as merge ranks in these vocabularies)."""
from __future__ import annotations
import codecs, re, unicodedata
from typing import Callable, Iterable

PRESETS = ("llama3", "llama-v3", "llama-bpe", "qwen2", "olmo", "kimi-k2", "tekken", "glm4")
_PRESET_ALIAS = {"qwen35": "qwen2", "qwen35moe": "qwen2"}
_LAST_LNZ = 0x323AF                   # highest code point in the Unicode categories L / N / Z

def _gpt2_byte_alphabet() -> dict[str, int]:
  """The printable stand-in character GPT-2 style vocabularies use for every byte: bytes that are printable Latin-1 stand for themselves,
  the other 68 are numbered from U+0100 on in byte order."""
  keep = set(range(0x21, 0x7F)) | set(range(0xA1, 0xAD)) | set(range(0xAE, 0x100))
  table, spill = {}, 0
  for b in range(256):
    if b in keep: table[chr(b)] = b
    else: table[chr(0x100 + spill)] = b; spill += 1
  return table

def _category_class(prefix: str) -> str:
  """Character-class body (escaped ranges) of all code points whose general category starts with `prefix`."""
  out, start, prev = [], None, None
  for cp in range(_LAST_LNZ + 2):
    inside = cp <= _LAST_LNZ and unicodedata.category(chr(cp)).startswith(prefix)
    if inside and start is None: start = cp
    if not inside and start is not None:
      out.append(re.escape(chr(start)) + ("-" + re.escape(chr(prev)) if prev != start else ""))
      start = None
    prev = cp
  return "".join(out)

_WORD_RE = None
def _word_pattern() -> re.Pattern:
  global _WORD_RE
  if _WORD_RE is None:
    ws, num, let = r"\t\n\x0b\x0c\r\x85" + _category_class("Z"), _category_class("N"), _category_class("L")
    alternatives = ["(?i:'s|'t|'re|'ve|'m|'ll|'d)", f"[^\\r\\n{num}{let}]?[{let}]+", f"[{num}]{{1,3}}", f" ?[^{ws}{num}{let}]+[\\r\\n]*",
                    f"[{ws}]*[\\r\\n]+", f"[{ws}]+(?![^{ws}])", f"[{ws}]+"]
    _WORD_RE = re.compile("|".join(alternatives))
  return _WORD_RE

class SimpleTokenizer:
  def __init__(self, normal_tokens: dict[str, int], special_tokens: dict[str, int], preset: str = "llama3", bos_id: int | None = None, eos_id: int = 0,
               eot_id: int | None = None):
    preset = _PRESET_ALIAS.get(preset, preset)
    if preset not in PRESETS: raise ValueError(f"Invalid tokenizer preset '{preset}'")
    alphabet = _gpt2_byte_alphabet()
    self._split_to_word = _word_pattern()
    self._specials = dict(special_tokens)
    self._special_re = re.compile("|".join(map(re.escape, self._specials))) if self._specials else None
    self._ids = {bytes(alphabet[ch] for ch in text): tid for text, tid in normal_tokens.items()}          # token bytes -> id
    self._bytes_of = {tid: raw for raw, tid in self._ids.items()}
    self._bytes_of.update({tid: text.encode() for text, tid in self._specials.items()})
    self.preset, self.bos_id, self.eos_id, self.eot_id = preset, bos_id, eos_id, eot_id

  @staticmethod
  def from_gguf_kv(kv: dict) -> "SimpleTokenizer":
    """tokenizer.ggml.tokens with token_type 1 are ordinary entries, every other type is matched as a literal special token (cli.py:41-49)."""
    types = kv["tokenizer.ggml.token_type"]
    normal = {t: i for i, t in enumerate(kv["tokenizer.ggml.tokens"]) if types[i] == 1}
    special = {t: i for i, t in enumerate(kv["tokenizer.ggml.tokens"]) if types[i] != 1}
    bos = kv.get("tokenizer.ggml.bos_token_id") if kv.get("tokenizer.ggml.add_bos_token", True) else None
    return SimpleTokenizer(normal, special, kv["tokenizer.ggml.pre"], bos_id=bos, eos_id=kv.get("tokenizer.ggml.eos_token_id", 0),
                           eot_id=kv.get("tokenizer.ggml.eot_token_id", special.get("<|im_end|>")))

  def _encode_word(self, word: bytes) -> list[int]:
    whole = self._ids.get(word)
    if whole is not None: return [whole]
    pieces = [word[i:i + 1] for i in range(len(word))]
    while len(pieces) > 1:
      best_rank, best_at = None, -1
      for at in range(len(pieces) - 1):                      # the leftmost pair of the lowest rank
        rank = self._ids.get(pieces[at] + pieces[at + 1])
        if rank is not None and (best_rank is None or rank < best_rank): best_rank, best_at = rank, at
      if best_at < 0: break
      pieces[best_at:best_at + 2] = [pieces[best_at] + pieces[best_at + 1]]
    try: return [self._ids[p] for p in pieces]
    except KeyError: raise RuntimeError("token not found") from None

  def _encode_plain(self, text: str) -> list[int]:
    return [t for word in self._split_to_word.findall(text) for t in self._encode_word(word.encode())]

  def encode(self, text: str) -> list[int]:
    if self._special_re is None: return self._encode_plain(text)
    out, at = [], 0
    for m in self._special_re.finditer(text):
      out += self._encode_plain(text[at:m.start()]); out.append(self._specials[m.group(0)]); at = m.end()
    return out + self._encode_plain(text[at:])

  def decode(self, ids: Iterable[int]) -> str: return b"".join(self._bytes_of[t] for t in ids).decode(errors="replace")

  def stream_decoder(self) -> Callable[..., str]:
    """Incremental decoding: bytes of a character split over tokens are held back until it is complete; call without an id to flush."""
    inc = codecs.getincrementaldecoder("utf-8")("replace")
    def step(tid: int | None = None) -> str: return inc.decode(b"", final=True) if tid is None else inc.decode(self._bytes_of[tid])
    return step

  def is_end(self, token_id: int) -> bool: return token_id in (self.eos_id, self.eot_id)
