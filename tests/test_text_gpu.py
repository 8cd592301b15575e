"""Text in, text out on the GPU: chat messages through Engine.generate, `--prompt TEXT` on the command
line with a tokenizer.json beside the weights, `--random-weights SEED` with a folder that holds only
a config.json, and a tokenizer that does not fit the model."""

import shutil
import subprocess
import sys
from pathlib import Path

import pytest
import torch

from tests.helpers import TINY_B
from tests.plain import model as plain
from tests.text_helpers import write_tiny_tokenizer

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parents[1]


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.weights import write_model_dir

    folder = tmp_path_factory.mktemp("text_b")
    write_model_dir(config_from_dict(TINY_B), seed=51, model_dir=folder, init="scaled")
    write_tiny_tokenizer(folder, 300)
    return folder


def plain_answer(folder, prompt_ids, new_tokens, stop):
    cfg, weights = plain.load_model_dir(folder, torch.float64)
    ids = list(prompt_ids)
    for _ in range(new_tokens):
        ids.append(int(plain.qwen3_forward(weights, cfg, ids)[-1].argmax()))
        if ids[-1] in stop:
            break
    return ids[len(prompt_ids):]


def test_chat_messages_through_the_engine(folder):
    from llm_runtime_study_amd import ChatMessage, Engine
    from llm_runtime_study_amd.text import format_qwen3_chat

    engine = Engine.from_model_dir(folder, dtype="float32", max_seq_len=128, max_batch_size=2)
    assert engine.tokenizer is not None and engine.tokenizer.chat_template is format_qwen3_chat
    messages = [ChatMessage("system", "Be concise."), ChatMessage("user", "hello world")]
    events = [e for _, e in engine.generate([messages], max_new_tokens=12)]
    prompt_ids = engine.tokenizer.encode(format_qwen3_chat(messages))
    expected = plain_answer(folder, prompt_ids, 12, TINY_B["eos_token_id"])
    assert [e.token_id for e in events] == expected and events[0].prompt_token_count == len(prompt_ids)
    # the deltas add up to the text, which is what decoding all tokens at once gives, up to bytes at the end that are
    # no whole character yet (a random model writes many such) and are held back
    text = engine.tokenizer.decode(expected, skip_special_tokens=True)
    assert "".join(e.text_delta for e in events) == events[-1].text
    assert text.startswith(events[-1].text) and set(text[len(events[-1].text):]) <= {"\ufffd"}
    thinking = [e for _, e in engine.generate([messages], max_new_tokens=2, enable_thinking=True)]
    assert thinking[0].prompt_token_count == len(engine.tokenizer.encode(format_qwen3_chat(messages, enable_thinking=True)))


def test_text_prompt_on_the_command_line(folder):
    from llm_runtime_study_amd.text import ChatMessage, TextTokenizer, format_qwen3_chat

    tokenizer = TextTokenizer.from_model_dir(folder, TINY_B["vocab_size"], format_qwen3_chat)
    prompt_ids = tokenizer.encode(format_qwen3_chat([ChatMessage("user", "the cat sat")]))
    expected = plain_answer(folder, prompt_ids, 10, TINY_B["eos_token_id"])
    streamed = tokenizer.decode(expected, skip_special_tokens=True)
    proc = subprocess.run([sys.executable, "-m", "llm_runtime_study_amd", "--model", str(folder), "--prompt", "the cat sat",
                           "--max-new-tokens", "10", "--max-seq-len", "128", "--dtype", "float32", "--device", "hip"],
                          cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    answer, _, metrics = proc.stdout.partition("\n\nmetrics\n")
    assert streamed.startswith(answer) and set(streamed[len(answer):]) <= {"\ufffd"}
    assert f"  prompt tokens:       {len(prompt_ids)}\n" in metrics and f"  generated tokens:    {len(expected)}\n" in metrics
    assert "  device:              cuda:0\n" in metrics and "  dtype:               torch.float32\n" in metrics
    assert "  decode throughput:   " in metrics and "  stop reason:         " in metrics and "  load time:           " in metrics
    # not streamed: the same text in one piece
    proc = subprocess.run([sys.executable, "-m", "llm_runtime_study_amd", "--model", str(folder), "--prompt", "the cat sat",
                           "--max-new-tokens", "10", "--max-seq-len", "128", "--dtype", "float32", "--no-stream", "--no-metrics"],
                          cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0 and proc.stdout == answer + "\n"


def test_random_weights_for_a_folder_with_a_configuration_only(folder, tmp_path):
    bare = tmp_path / "bare"
    bare.mkdir()
    shutil.copy(folder / "config.json", bare / "config.json")
    command = [sys.executable, "-m", "llm_runtime_study_amd", "--model", str(bare), "--prompt-ids", "5,6,7", "--max-new-tokens", "6",
               "--max-seq-len", "64", "--no-metrics"]
    first = subprocess.run(command + ["--random-weights", "3"], cwd=ROOT, capture_output=True, text=True, timeout=300)
    again = subprocess.run(command + ["--random-weights", "3"], cwd=ROOT, capture_output=True, text=True, timeout=300)
    other = subprocess.run(command + ["--random-weights", "4"], cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert first.returncode == 0, first.stderr[-2000:]
    tokens = first.stdout.split()
    assert 1 <= len(tokens) <= 6 and all(0 <= int(t) < TINY_B["vocab_size"] for t in tokens)
    assert again.stdout == first.stdout and other.returncode == 0 and other.stdout != first.stdout
    missing = subprocess.run(command, cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert missing.returncode == 2 and "error: " in missing.stderr and "model.safetensors" in missing.stderr


def test_a_tokenizer_that_does_not_fit_the_model_is_refused(folder, tmp_path):
    from llm_runtime_study_amd import Engine
    from llm_runtime_study_amd.errors import TokenizerError

    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.weights import write_model_dir

    small = tmp_path / "small"
    write_model_dir(config_from_dict(dict(TINY_B, vocab_size=290)), seed=52, model_dir=small, init="scaled")
    shutil.copy(folder / "tokenizer.json", small / "tokenizer.json")           # 300 entries for a model of 290
    with pytest.raises(TokenizerError, match="more entries than the model output vocabulary: 300 > 290"):
        Engine.from_model_dir(small, dtype="float32", max_seq_len=64)
