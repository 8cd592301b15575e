"""Thin wrapper around a model folder's tokenizer.json (reference mini_llm/tokenizer.py:68-154).

The tokenizer is optional: benchmarks and tests feed token ids.  Text prompts need the
`tokenizers` package and a tokenizer.json next to the weights.
"""

from __future__ import annotations

from pathlib import Path
from typing import Sequence

from ..errors import TokenizerError
from .chat import ChatMessage, format_qwen3_chat


class TextTokenizer:
    def __init__(self, tokenizer, model_vocab_size: int):
        size = tokenizer.get_vocab_size(with_added_tokens=True)
        if size > model_vocab_size:
            raise TokenizerError(
                f"tokenizer contains more entries than the model output vocabulary: {size} > {model_vocab_size}")
        self._tokenizer = tokenizer
        self.model_vocab_size = model_vocab_size

    @classmethod
    def from_model_dir(cls, model_dir, model_vocab_size: int) -> "TextTokenizer | None":
        """The folder's tokenizer, or None when it ships none."""
        path = Path(model_dir) / "tokenizer.json"
        if not path.is_file():
            return None
        try:
            from tokenizers import Tokenizer
        except ImportError as exc:
            raise TokenizerError("the `tokenizers` package is needed to read tokenizer.json") from exc
        try:
            tokenizer = Tokenizer.from_file(str(path))
        except Exception as exc:
            raise TokenizerError(f"could not load tokenizer: {path}") from exc
        return cls(tokenizer, model_vocab_size)

    def encode(self, text: str) -> list[int]:
        if not isinstance(text, str):
            raise TokenizerError(f"text must be str, got {type(text).__name__}")
        return self._tokenizer.encode(text, add_special_tokens=False).ids

    def decode(self, token_ids: Sequence[int], *, skip_special_tokens: bool = False) -> str:
        return self._tokenizer.decode(list(token_ids), skip_special_tokens=skip_special_tokens)

    def format_chat(self, messages: Sequence[ChatMessage], *, enable_thinking: bool = False) -> str:
        return format_qwen3_chat(messages, enable_thinking=enable_thinking)


class IncrementalTextDecoder:
    """Emits only text that is complete: a token ending inside a multi-byte character waits
    for the next one (reference mini_llm/generation.py:72-92)."""

    def __init__(self, tokenizer: TextTokenizer | None):
        self.tokenizer = tokenizer
        self.pending: list[int] = []
        self.text = ""

    def add(self, token_id: int) -> str:
        if self.tokenizer is None:
            return ""
        self.pending.append(token_id)
        piece = self.tokenizer.decode(self.pending, skip_special_tokens=True)
        if piece.endswith("�"):
            return ""
        self.pending.clear()
        self.text += piece
        return piece
