"""A model folder's tokenizer.json behind the few calls the runtime needs, and the piecewise
decoding of generated tokens into text.

The tokenizer is optional: benchmarks and tests feed token ids.  Text prompts need the `tokenizers`
package and a tokenizer.json next to the weights (reference mini_llm/tokenizer.py:68-154).  Which chat
template turns messages into prompt text is the architecture's business: the wrapper is handed the
template of the architecture registry's entry and knows none itself.
"""

from __future__ import annotations

from pathlib import Path
from typing import Callable, Sequence

from ..errors import TokenizerError
from .chat import ChatMessage

REPLACEMENT = "�"   # what a decoder puts where a byte sequence is not yet a whole character


class TextTokenizer:
    def __init__(self, tokenizer, model_vocab_size: int, chat_template: Callable | None = None):
        entries = tokenizer.get_vocab_size(with_added_tokens=True)
        if entries > model_vocab_size:
            raise TokenizerError(
                f"tokenizer contains more entries than the model output vocabulary: {entries} > {model_vocab_size}")
        self._tokenizer = tokenizer
        self.model_vocab_size = model_vocab_size
        self.chat_template = chat_template

    @classmethod
    def from_model_dir(cls, model_dir, model_vocab_size: int, chat_template: Callable | None = None) -> "TextTokenizer | None":
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
        return cls(tokenizer, model_vocab_size, chat_template)

    def encode(self, text: str) -> list[int]:
        if not isinstance(text, str):
            raise TokenizerError(f"text must be str, got {type(text).__name__}")
        return self._tokenizer.encode(text, add_special_tokens=False).ids

    def decode(self, token_ids: Sequence[int], *, skip_special_tokens: bool = False) -> str:
        return self._tokenizer.decode(list(token_ids), skip_special_tokens=skip_special_tokens)

    def format_chat(self, messages: Sequence[ChatMessage], *, enable_thinking: bool = False) -> str:
        if self.chat_template is None:
            raise TokenizerError("this model's architecture registers no chat template; pass token ids or plain text")
        return self.chat_template(messages, enable_thinking=enable_thinking)


class TextStream:
    """Generated token ids in, text out, a piece at a time.

    A byte-level vocabulary may cut a character of several bytes between two tokens; decoding the
    first alone gives the replacement character.  push() therefore decodes the tokens not yet turned
    into text together and hands out their text only once it no longer ends in a replacement
    character; until then they wait.  `text` is everything handed out so far.  Without a tokenizer
    every piece is empty.  (Behaviour of the reference's streaming decoder, mini_llm/generation.py:72-92.)"""

    def __init__(self, tokenizer: TextTokenizer | None):
        self._tokenizer = tokenizer
        self._waiting: list[int] = []
        self._pieces: list[str] = []

    @property
    def text(self) -> str:
        return "".join(self._pieces)

    def push(self, token_id: int) -> str:
        if self._tokenizer is None:
            return ""
        self._waiting.append(token_id)
        piece = self._tokenizer.decode(self._waiting, skip_special_tokens=True)
        if piece.endswith(REPLACEMENT):
            return ""
        self._waiting = []
        self._pieces.append(piece)
        return piece
