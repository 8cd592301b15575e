"""Chat messages, the rules a conversation must keep, and the Qwen3 template.

A chat template is a function (messages, *, enable_thinking=False, add_generation_prompt=True) -> str;
each architecture names its own in the architecture registry (config/registry.py), and the tokenizer
wrapper is handed it, so another architecture brings another template without touching this package's
text code.  Reference mini_llm/chat.py:23-58 (the rules), 87-112 (the Qwen3 format, pinned by
tests/test_tokenizer.py:24-75 there).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Sequence

from ..errors import TokenizerError

TURN_ROLES = ("user", "assistant")


@dataclass(frozen=True)
class ChatMessage:
    role: str       # "system" (first message only), "user" or "assistant"
    content: str


def validate_chat_messages(messages: Sequence[ChatMessage], *, add_generation_prompt: bool = True) -> None:
    """An optional system message first, then user and assistant taking turns, the user beginning; when
    the model is to answer (`add_generation_prompt`), the user must have spoken last."""
    if not messages:
        raise TokenizerError("chat requires at least one message")
    turn = 0   # index into TURN_ROLES of the role that must speak next
    for index, message in enumerate(messages):
        if not isinstance(message, ChatMessage):
            raise TokenizerError(f"message {index} must be ChatMessage, got {type(message).__name__}")
        if not isinstance(message.content, str):
            raise TokenizerError(f"message {index} content must be str")
        if message.role == "system":
            if index:
                raise TokenizerError("a system message is only allowed as the first turn")
        elif message.role not in TURN_ROLES:
            raise TokenizerError(f"unsupported chat role at message {index}: {message.role!r}")
        elif message.role != TURN_ROLES[turn]:
            raise TokenizerError(f"expected {TURN_ROLES[turn]!r} at message {index}, got {message.role!r}")
        else:
            turn ^= 1
    if add_generation_prompt and messages[-1].role != "user":
        raise TokenizerError("the final message must have role 'user' when adding a generation prompt")


def format_qwen3_chat(messages: Sequence[ChatMessage], *, enable_thinking: bool = False,
                      add_generation_prompt: bool = True) -> str:
    """`<|im_start|>{role}\\n{content}<|im_end|>\\n` for every message; then, if the model is to answer,
    the assistant's header and, with thinking off, an empty think block."""
    validate_chat_messages(messages, add_generation_prompt=add_generation_prompt)
    pieces = [f"<|im_start|>{m.role}\n{m.content}<|im_end|>\n" for m in messages]
    if add_generation_prompt:
        pieces.append("<|im_start|>assistant\n" if enable_thinking else "<|im_start|>assistant\n<think>\n\n</think>\n\n")
    return "".join(pieces)
