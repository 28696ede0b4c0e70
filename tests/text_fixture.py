"""A small synthetic byte-level BPE tokenizer for the tests: the 256 byte symbols, a few merged
words, and the Qwen3 special tokens, written as tokenizer.json or as the reference's three
files.  Ids are small so that a tiny model's vocabulary covers them."""
import json
import os

from zinfer_amd.text.bpe import byte_table

WORDS = ["Hello", " hello", "user", "assistant", "test", "\n\n", " world", "Hi", "system"]
SPECIALS = ["<|endoftext|>", "<|im_start|>", "<|im_end|>", "<think>", "</think>"]


def build():
    """(vocab, merges, specials): words are merged left to right, one symbol at a time."""
    enc, _ = byte_table()
    vocab = {enc[b]: b for b in range(256)}
    merges = []
    for w in WORDS:
        symbols = [enc[b] for b in w.encode("utf-8")]
        left = symbols[0]
        for s in symbols[1:]:
            pair = left + " " + s
            if pair not in merges:
                merges.append(pair)
            left = left + s
            vocab.setdefault(left, len(vocab))
    specials = {}
    for s in SPECIALS:
        specials[s] = len(vocab) + len(specials)
    return vocab, merges, specials


def write_tokenizer_json(folder: str) -> None:
    vocab, merges, specials = build()
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "tokenizer.json"), "w", encoding="utf-8") as f:
        json.dump({"model": {"type": "BPE", "vocab": vocab, "merges": merges},
                   "added_tokens": [{"id": i, "content": s, "special": True}
                                    for s, i in specials.items()]}, f, ensure_ascii=False)


def write_reference_files(folder: str) -> None:
    vocab, merges, specials = build()
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "vocab.json"), "w", encoding="utf-8") as f:
        json.dump(vocab, f, ensure_ascii=False)
    with open(os.path.join(folder, "merges.txt"), "w", encoding="utf-8") as f:
        f.write("#version: 0.2\n" + "\n".join(merges) + "\n")
    with open(os.path.join(folder, "tokenizer_config.json"), "w", encoding="utf-8") as f:
        json.dump({"added_tokens_decoder": {str(i): {"content": s} for s, i in specials.items()}}, f)
