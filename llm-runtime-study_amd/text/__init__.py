"""Chat messages and templates, the tokenizer wrapper and streamed detokenisation."""

from .chat import ChatMessage, format_qwen3_chat, validate_chat_messages
from .tokenizer import TextStream, TextTokenizer

__all__ = ["ChatMessage", "TextStream", "TextTokenizer", "format_qwen3_chat", "validate_chat_messages"]
