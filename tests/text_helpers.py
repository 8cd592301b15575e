"""A tiny byte-level BPE tokenizer.json, built with the `tokenizers` package for the text tests."""

from __future__ import annotations

from pathlib import Path

SPECIALS = ["<|endoftext|>", "<|im_start|>", "<|im_end|>"]
PLAIN_ADDED = ["<think>", "</think>"]
CORPUS = ["hello world", "Hello there, hello again", "the cat sat on the mat", "system user assistant", "Be concise.",
          "one two three", "Solve this", "world of words"] * 4


def write_tiny_tokenizer(folder, vocab_size: int = 300) -> Path:
    """Writes <folder>/tokenizer.json: the 256 byte symbols, a few merges learnt from ASCII text (so that
    a character of several bytes is always cut into single-byte tokens), the ChatML control tokens as
    special tokens and the think tags as ordinary added tokens, `vocab_size` entries in all."""
    from tokenizers import Tokenizer, decoders, models, pre_tokenizers, trainers

    tokenizer = Tokenizer(models.BPE())
    tokenizer.pre_tokenizer = pre_tokenizers.ByteLevel(add_prefix_space=False, use_regex=True)
    tokenizer.decoder = decoders.ByteLevel()
    trainer = trainers.BpeTrainer(vocab_size=vocab_size - len(SPECIALS) - len(PLAIN_ADDED), special_tokens=[],
                                  initial_alphabet=pre_tokenizers.ByteLevel.alphabet(), show_progress=False)
    tokenizer.train_from_iterator(CORPUS, trainer)
    tokenizer.add_special_tokens(SPECIALS)
    tokenizer.add_tokens(PLAIN_ADDED)
    path = Path(folder) / "tokenizer.json"
    tokenizer.save(str(path))
    return path
