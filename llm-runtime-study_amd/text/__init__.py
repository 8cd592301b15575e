"""Chat template and tokenizer wrapper."""

from .chat import ChatMessage, format_qwen3_chat
from .tokenizer import IncrementalTextDecoder, TextTokenizer

__all__ = ["ChatMessage", "IncrementalTextDecoder", "TextTokenizer", "format_qwen3_chat"]
