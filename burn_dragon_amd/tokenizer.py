"""Tokenizers of the reference (src/tokenizer/mod.rs:17-27 trait; byte.rs; char_vocab.rs).

Host-side text <-> token ids; nothing here touches the GPU."""
from __future__ import annotations

import json
from typing import Dict, Iterable, List, Optional

PAD_CHAR, BOS_CHAR, EOS_CHAR, UNK_CHAR = "\u0000", "\u0001", "\u0002", "\u0003"
BYTE_VOCAB_SIZE = 256


class Tokenizer:
    """src/tokenizer/mod.rs:17-27."""

    def encode(self, text: str, add_bos: bool = False, add_eos: bool = False) -> List[int]:
        raise NotImplementedError

    def decode(self, ids: Iterable[int]) -> str:
        raise NotImplementedError

    def __len__(self) -> int:
        raise NotImplementedError

    def is_empty(self) -> bool:
        return len(self) == 0

    def bos_id(self) -> Optional[int]:
        return None

    def eos_id(self) -> Optional[int]:
        return None

    def pad_id(self) -> Optional[int]:
        return None

    def unk_id(self) -> Optional[int]:
        return None


class ByteTokenizer(Tokenizer):
    """src/tokenizer/byte.rs: ids 0..255 are the utf-8 bytes; with special tokens bos=256, eos=257,
    pad=258 and the vocabulary has 259 entries (:14-37)."""

    def __init__(self, add_special_tokens: bool = False):
        self.add_special_tokens = add_special_tokens
        self.bos = self.eos = self.pad = None
        self.vocab_size = BYTE_VOCAB_SIZE
        if add_special_tokens:
            self.bos, self.eos, self.pad = 256, 257, 258
            self.vocab_size = 259

    def encode(self, text, add_bos=False, add_eos=False):  # :40-55
        tokens = []
        if add_bos and self.bos is not None:
            tokens.append(self.bos)
        tokens.extend(text.encode("utf-8"))
        if add_eos and self.eos is not None:
            tokens.append(self.eos)
        return tokens

    def decode(self, ids):  # :57-71 — pad/bos skipped, stops at eos, ids >= 256 dropped, lossy utf-8
        out = bytearray()
        for i in ids:
            if i == self.pad and self.pad is not None or i == self.bos and self.bos is not None:
                continue
            if self.eos is not None and i == self.eos:
                break
            if 0 <= i < BYTE_VOCAB_SIZE:
                out.append(i)
        return out.decode("utf-8", errors="replace")

    def __len__(self):
        return self.vocab_size

    def bos_id(self):
        return self.bos

    def eos_id(self):
        return self.eos

    def pad_id(self):
        return self.pad

    def __eq__(self, other):
        return isinstance(other, ByteTokenizer) and self.add_special_tokens == other.add_special_tokens


class CharVocab(Tokenizer):
    """src/tokenizer/char_vocab.rs: one id per character in first-seen order after the specials
    pad=U+0000, bos=U+0001, eos=U+0002 and (optionally) unk=U+0003."""

    def __init__(self, chars: List[str], include_unknown: bool):  # from_chars :47-88
        if not chars:
            raise ValueError("vocabulary cannot be empty")
        self.id2ch: List[str] = []
        self.ch2id: Dict[str, int] = {}
        for idx, ch in enumerate(chars):
            if len(ch) != 1:
                raise ValueError(f"vocabulary entry {ch!r} is not a single character")
            if ch in self.ch2id:
                raise ValueError(f"duplicate character {ch!r}")
            self.ch2id[ch] = idx
            self.id2ch.append(ch)
        for name, ch in (("BOS", BOS_CHAR), ("EOS", EOS_CHAR), ("PAD", PAD_CHAR)):
            if ch not in self.ch2id:
                raise ValueError(f"missing {name} character in vocabulary")
        self.bos, self.eos, self.pad = self.ch2id[BOS_CHAR], self.ch2id[EOS_CHAR], self.ch2id[PAD_CHAR]
        self.unk = self.ch2id.get(UNK_CHAR) if include_unknown else None

    @classmethod
    def fit(cls, texts: Iterable[str], include_unknown: bool = True) -> "CharVocab":  # :28-45
        chars = [PAD_CHAR, BOS_CHAR, EOS_CHAR] + ([UNK_CHAR] if include_unknown else [])
        seen = set(chars)
        for text in texts:
            for ch in text:
                if ch not in seen:
                    seen.add(ch)
                    chars.append(ch)
        return cls(chars, include_unknown)

    def to_record(self) -> dict:  # :90-98
        return {"chars": list(self.id2ch), "bos": self.bos, "eos": self.eos, "pad": self.pad, "unk": self.unk}

    @classmethod
    def from_record(cls, record: dict) -> "CharVocab":  # :100-110 — the stored ids win over the derived ones
        vocab = cls(list(record["chars"]), record.get("unk") is not None)
        vocab.bos, vocab.eos, vocab.pad, vocab.unk = record["bos"], record["eos"], record["pad"], record.get("unk")
        return vocab

    @classmethod
    def from_json_str(cls, data: str) -> "CharVocab":  # :136-140
        return cls.from_record(json.loads(data))

    @classmethod
    def from_json_bytes(cls, data: bytes) -> "CharVocab":  # :142-146
        return cls.from_json_str(data.decode("utf-8"))

    @classmethod
    def load(cls, path: str) -> "CharVocab":  # :124-134
        with open(path, "r", encoding="utf-8") as f:
            return cls.from_json_str(f.read())

    def save(self, path: str) -> None:  # :112-122
        with open(path, "w", encoding="utf-8") as f:
            json.dump(self.to_record(), f, indent=2, ensure_ascii=False)

    def encode(self, text, add_bos=False, add_eos=False):  # :148-176
        tokens = [self.bos] if add_bos else []
        for ch in text:
            idx = self.ch2id.get(ch)
            if idx is None:
                if self.unk is None:
                    raise KeyError(f"character {ch!r} missing from vocabulary and no <unk> token configured")
                idx = self.unk
            tokens.append(idx)
        if add_eos:
            tokens.append(self.eos)
        return tokens

    def decode(self, ids):  # :178-203 — pad/bos skipped, stops at eos, unk printed as '?'
        out = []
        for i in ids:
            if not 0 <= i < len(self.id2ch):
                raise IndexError(f"token id {i} out of range")
            if i == self.pad or i == self.bos:
                continue
            if i == self.eos:
                break
            out.append("?" if self.unk is not None and i == self.unk else self.id2ch[i])
        return "".join(out)

    def __len__(self):
        return len(self.id2ch)

    def contains(self, ch: str) -> bool:
        return ch in self.ch2id

    def bos_id(self):
        return self.bos

    def eos_id(self):
        return self.eos

    def pad_id(self):
        return self.pad

    def unk_id(self):
        return self.unk

    def __eq__(self, other):
        return isinstance(other, CharVocab) and self.to_record() == other.to_record()
