"""Text in, text out on the CPU: the chat template's vectors, the tokenizer wrapper, streamed
detokenisation across a character cut between tokens, the template's place in the architecture
registry, and a scheduler run from chat messages to text deltas with a fake step function."""

import pytest
import torch

from llm_runtime_study_amd.config import chat_template_for, config_from_dict, register_architecture
from llm_runtime_study_amd.errors import ConfigError, GenerationError, TokenizerError
from llm_runtime_study_amd.text import ChatMessage, TextStream, TextTokenizer, format_qwen3_chat
from tests.helpers import TINY_B
from tests.text_helpers import write_tiny_tokenizer


@pytest.fixture(scope="module")
def tokenizer(tmp_path_factory):
    folder = tmp_path_factory.mktemp("tokenizer")
    write_tiny_tokenizer(folder, 300)
    return TextTokenizer.from_model_dir(folder, 331, format_qwen3_chat)


# ----------------------------------------------------------------- chat template
def test_chat_vectors_of_the_reference():
    # reference tests/test_tokenizer.py:24-39
    assert format_qwen3_chat([ChatMessage("system", "Be concise."), ChatMessage("user", "Hello")], enable_thinking=False) == (
        "<|im_start|>system\nBe concise.<|im_end|>\n"
        "<|im_start|>user\nHello<|im_end|>\n"
        "<|im_start|>assistant\n<think>\n\n</think>\n\n")
    # :41-48 thinking on: the prompt ends after the assistant header
    thinking = format_qwen3_chat([ChatMessage("user", "Solve this")], enable_thinking=True)
    assert thinking.endswith("<|im_start|>assistant\n") and "<think>" not in thinking
    # :50-59 an assistant turn in the history
    history = format_qwen3_chat([ChatMessage("user", "one"), ChatMessage("assistant", "two"), ChatMessage("user", "three")])
    assert "<|im_start|>assistant\ntwo<|im_end|>\n" in history
    # :61-67 history only
    assert format_qwen3_chat([ChatMessage("user", "one"), ChatMessage("assistant", "two")], add_generation_prompt=False).endswith("two<|im_end|>\n")


def test_conversations_out_of_order_are_refused():
    # reference tests/test_tokenizer.py:69-80 and mini_llm/chat.py:23-58
    with pytest.raises(TokenizerError, match="expected 'assistant'"):
        format_qwen3_chat([ChatMessage("user", "one"), ChatMessage("user", "two")])
    with pytest.raises(TokenizerError, match="final message"):
        format_qwen3_chat([ChatMessage("user", "one"), ChatMessage("assistant", "two")])
    with pytest.raises(TokenizerError, match="at least one message"):
        format_qwen3_chat([])
    with pytest.raises(TokenizerError, match="only allowed as the first turn"):
        format_qwen3_chat([ChatMessage("user", "one"), ChatMessage("system", "late")])
    with pytest.raises(TokenizerError, match="unsupported chat role at message 0: 'tool'"):
        format_qwen3_chat([ChatMessage("tool", "x")])
    with pytest.raises(TokenizerError, match="expected 'user' at message 1"):
        format_qwen3_chat([ChatMessage("system", "s"), ChatMessage("assistant", "x")])
    with pytest.raises(TokenizerError, match="must be ChatMessage"):
        format_qwen3_chat(["hello"])
    with pytest.raises(TokenizerError, match="content must be str"):
        format_qwen3_chat([ChatMessage("user", 5)])


# -------------------------------------------------------------------- tokenizer
def test_formatted_prompt_round_trips_and_special_tokens_can_be_dropped(tokenizer):
    # what reference tests/test_tokenizer.py:160-180 checks on the real vocabulary, here on the tiny one
    prompt = tokenizer.format_chat([ChatMessage("user", "Hello")])
    ids = tokenizer.encode(prompt)
    im_start, im_end = tokenizer.encode("<|im_start|>"), tokenizer.encode("<|im_end|>")
    assert len(im_start) == 1 and len(im_end) == 1 and ids[0] == im_start[0] and im_end[0] in ids
    assert tokenizer.decode(ids) == prompt
    plain = tokenizer.decode(ids, skip_special_tokens=True)
    assert "<|im_start|>" not in plain and "<|im_end|>" not in plain and "<think>" in plain
    assert all(0 <= t < 300 for t in ids)
    with pytest.raises(TokenizerError, match="text must be str"):
        tokenizer.encode(5)


def test_a_tokenizer_larger_than_the_model_vocabulary_is_refused(tmp_path):
    write_tiny_tokenizer(tmp_path, 300)
    with pytest.raises(TokenizerError, match="more entries than the model output vocabulary: 300 > 299"):
        TextTokenizer.from_model_dir(tmp_path, 299)
    assert TextTokenizer.from_model_dir(tmp_path, 300) is not None
    assert TextTokenizer.from_model_dir(tmp_path / "nothing here", 300) is None
    (tmp_path / "tokenizer.json").write_text("{ not json")
    with pytest.raises(TokenizerError, match="could not load tokenizer"):
        TextTokenizer.from_model_dir(tmp_path, 300)


def test_a_character_cut_between_tokens_waits_for_its_last_byte(tokenizer):
    # reference mini_llm/generation.py:72-92
    text = "hello é world 🙂!"
    ids = tokenizer.encode(text)
    assert tokenizer.decode(ids) == text
    cut = tokenizer.encode("é")
    assert len(cut) == 2 and tokenizer.decode(cut[:1]).endswith("�")       # the tiny vocabulary has no merge for it
    stream = TextStream(tokenizer)
    pieces = [stream.push(t) for t in ids]
    assert "".join(pieces) == text and stream.text == text
    assert all("�" not in piece for piece in pieces)
    at = ids.index(cut[0])
    assert pieces[at] == "" and pieces[at + 1] == "é"                            # held back, then whole
    face = tokenizer.encode("🙂")
    start = next(i for i in range(len(ids)) if ids[i:i + len(face)] == face)
    assert len(face) == 4 and pieces[start:start + 4] == ["", "", "", "🙂"]
    # special tokens leave no text, and without a tokenizer there is none at all
    stream = TextStream(tokenizer)
    assert stream.push(tokenizer.encode("<|im_end|>")[0]) == "" and stream.text == ""
    silent = TextStream(None)
    assert silent.push(5) == "" and silent.text == ""


# --------------------------------------------------------- registry and protocol
def test_the_chat_template_comes_from_the_architecture_registry(tokenizer):
    config = config_from_dict(TINY_B)
    assert chat_template_for(config) is format_qwen3_chat

    class OtherConfig:
        model_type = "other"
        vocab_size = 10
        eos_token_ids = (1,)

        @classmethod
        def from_dict(cls, raw):
            return cls()

        def validate_context_length(self, max_seq_len):
            pass

        def to_json_dict(self):
            return {"architectures": ["OtherForCausalLM"]}

    def shout(messages, *, enable_thinking=False):
        return "".join(f"[{m.role.upper()}] {m.content}\n" for m in messages)

    register_architecture("OtherForCausalLM", OtherConfig, lambda config: None, chat_template=shout)
    other = config_from_dict({"architectures": ["OtherForCausalLM"]})
    assert chat_template_for(other) is shout
    wrapper = TextTokenizer(tokenizer._tokenizer, 331, chat_template_for(other))
    assert wrapper.format_chat([ChatMessage("user", "hi")]) == "[USER] hi\n"
    register_architecture("BareForCausalLM", type("BareConfig", (OtherConfig,), {}), lambda config: None)
    bare = TextTokenizer(tokenizer._tokenizer, 331, chat_template_for(config_from_dict({"architectures": ["BareForCausalLM"]})))
    with pytest.raises(TokenizerError, match="registers no chat template"):
        bare.format_chat([ChatMessage("user", "hi")])


def test_a_configuration_class_must_provide_what_the_engine_reads():
    class Lacking:
        model_type = "x"
        vocab_size = 3

        @classmethod
        def from_dict(cls, raw):
            return cls()

    with pytest.raises(ConfigError, match="lacks: eos_token_ids, validate_context_length, to_json_dict"):
        register_architecture("LackingForCausalLM", Lacking, lambda config: None)
    with pytest.raises(ConfigError, match="must be callable"):
        register_architecture("X", type("C", (), {"model_type": "", "vocab_size": 1, "eos_token_ids": (), "from_dict": classmethod(lambda c, r: c()),
                                                  "validate_context_length": lambda s, n: None, "to_json_dict": lambda s: {}}), None)


# ------------------------------------------ chat messages through the scheduler
def test_chat_messages_become_token_ids_and_tokens_become_text_deltas(tokenizer):
    from llm_runtime_study_amd.engine.scheduler import generate
    from tests.test_scheduler import FakeRunner, scheduler

    answer = tokenizer.encode("hello é") + tokenizer.encode("<|im_end|>")
    eos = answer[-1]
    runner = FakeRunner({0: answer}, num_pages=32, page_size=4, max_seq_len=128)
    s = scheduler(runner, max_seq_len=128, max_step_tokens=16, eos_token_ids=(eos,), vocab_size=331, tokenizer=tokenizer)

    class Wide:      # the fake runner's logits must hold the tokenizer's ids
        def choose(self, logits, rows):
            return logits.argmax(-1).tolist()

    s.sampler = Wide()
    import tests.test_scheduler as fake
    old, fake.VOCAB = fake.VOCAB, 331
    try:
        events = [e for _, e in generate(s, [[ChatMessage("system", "Be concise."), ChatMessage("user", "Hello")]], max_new_tokens=20)]
    finally:
        fake.VOCAB = old
    prompt = tokenizer.encode(format_qwen3_chat([ChatMessage("system", "Be concise."), ChatMessage("user", "Hello")]))
    fed = [t for call in runner.calls for _, tokens, _ in call for t in tokens]
    assert fed[:len(prompt)] == prompt and events[0].prompt_token_count == len(prompt)
    assert "".join(e.text_delta for e in events) == "hello é" and events[-1].text == "hello é" and events[-1].finish_reason == "eos"
    assert [e.text_delta for e in events][-3:] == ["", "é", ""]       # first byte held back, the character, the silent end token
    # a model folder without tokenizer takes token ids only
    s = scheduler(FakeRunner({0: [1]}), tokenizer=None)
    with pytest.raises(GenerationError, match="needs a tokenizer"):
        s.add_request([ChatMessage("user", "hi")], max_new_tokens=2)
