"""Qwen3 chat template (reference mini_llm/chat.py:23-58 validation, 87-112 format)."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Sequence

from ..errors import TokenizerError

ROLES = ("system", "user", "assistant")


@dataclass(frozen=True)
class ChatMessage:
    role: str
    content: str


def validate_chat_messages(messages: Sequence[ChatMessage]) -> None:
    if not messages:
        raise TokenizerError("a chat prompt needs at least one message")
    for index, message in enumerate(messages):
        if not isinstance(message, ChatMessage):
            raise TokenizerError(f"message {index} must be a ChatMessage")
        if message.role not in ROLES:
            raise TokenizerError(f"message {index} has unsupported role {message.role!r}")
        if not isinstance(message.content, str):
            raise TokenizerError(f"message {index} content must be str")
        if message.role == "system" and index != 0:
            raise TokenizerError("a system message may only come first")
    if messages[-1].role != "user":
        raise TokenizerError("the last message must come from the user")


def format_qwen3_chat(messages: Sequence[ChatMessage], *, enable_thinking: bool = False) -> str:
    """<|im_start|>{role}\\n{content}<|im_end|>\\n per message, then the assistant header and,
    with thinking off, an empty think block."""
    validate_chat_messages(messages)
    prompt = "".join(f"<|im_start|>{m.role}\n{m.content}<|im_end|>\n" for m in messages)
    prompt += "<|im_start|>assistant\n"
    if not enable_thinking:
        prompt += "<think>\n\n</think>\n\n"
    return prompt
