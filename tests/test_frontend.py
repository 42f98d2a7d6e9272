"""The command line: options, chat rendering, streaming text (no GPU), and one run on a
tiny model with a tokenizer built here (GPU)."""
import json
import subprocess
import sys
from pathlib import Path

import pytest

from edge_infer_amd.frontend import chat
from helpers import make_folder

ROOT = Path(__file__).resolve().parents[1]


def test_option_names_and_defaults_follow_the_reference():
    """frontend/chat.py:82-96: --max_length is an alias of --max_new_tokens (424);
    temperature 0.7, top_p 1, top_k 20."""
    args = chat.build_parser().parse_args(["--model_path", "x"])
    assert (args.max_new_tokens, args.temperature, args.top_p, args.top_k) == (424, 0.7, 1.0, 20)
    assert args.model_type == "qwen3_bf16" and args.device == "cuda"
    assert args.context_capacity is None
    assert args.system_prompt == "You are a helpful AI assistant."
    assert chat.build_parser().parse_args(["--model_path", "x", "--max_length", "7"]).max_new_tokens == 7


def test_chat_rendering(tmp_path):
    messages = [{"role": "system", "content": "S"}, {"role": "user", "content": "hi"}]
    assert chat.render_chat(messages, tmp_path) == \
        "<|im_start|>system\nS<|im_end|>\n<|im_start|>user\nhi<|im_end|>\n<|im_start|>assistant\n"
    template = "{% for m in messages %}[{{ m.role }}:{{ m.content }}]{% endfor %}" \
               "{% if add_generation_prompt %}>{% endif %}"
    (tmp_path / "tokenizer_config.json").write_text(json.dumps({"chat_template": template}))
    assert chat.render_chat(messages, tmp_path) == "[system:S][user:hi]>"


def test_streaming_holds_back_incomplete_characters():
    class Bytes:
        """Tokens are single bytes of UTF-8 text; no description, so the stream decodes the
        whole answer again at every token."""
        def decode(self, ids, skip_special_tokens=True):
            return bytes(ids).decode("utf-8", errors="replace")
    stream = chat.TextStream(Bytes())
    shown = ""
    for byte in "a\u20acb\U0001f600".encode("utf-8"):   # 1, 3, 1 and 4 bytes
        piece = stream.push(byte)
        assert "\ufffd" not in piece
        shown += piece
    assert shown + stream.finish() == "a\u20acb\U0001f600" == stream.text
    # an answer that ends inside a character: the end hands out what there is
    stream = chat.TextStream(Bytes())
    assert stream.push(0x61) == "a" and stream.push(0xE2) == "" and stream.finish() == "\ufffd"


def test_streaming_of_a_byte_level_vocabulary_collects_bytes():
    """Characters spread over several tokens come out once complete, special tokens are
    not text, and what a cut-off answer leaves is handed out at the end."""
    from tokenizers import Tokenizer, decoders, models
    alphabet = {byte: char for char, byte in chat._byte_alphabet().items()}
    assert len(alphabet) == 256 and alphabet[ord("A")] == "A" and alphabet[0x20] == "\u0120"
    vocab = {char: index for index, char in enumerate(alphabet[b] for b in range(256))}
    vocab[alphabet[0xE2] + alphabet[0x82]] = 256            # two of the euro sign's three bytes
    tokenizer = Tokenizer(models.BPE(vocab=vocab, merges=[]))
    tokenizer.decoder = decoders.ByteLevel()
    tokenizer.add_special_tokens(["<|im_end|>"])
    end = tokenizer.token_to_id("<|im_end|>")
    stream = chat.TextStream(tokenizer)
    pieces = [stream.push(t) for t in (ord("h"), 0x20, 256, 0xAC, 0xF0, 0x9F, end, 0x98, 0x80)]
    assert pieces == ["h", " ", "", "\u20ac", "", "", "", "", "\U0001f600"]
    assert stream.finish() == "" and stream.text == "h \u20ac\U0001f600"
    assert [chat._whole_characters(data) for data in
            (b"", b"ab", b"a\xe2", b"a\xe2\x82", b"a\xe2\x82\xac", b"\xf0\x9f\x98", b"\x80\x80")] \
        == [0, 2, 1, 1, 4, 0, 2]


def make_word_tokenizer(folder, vocab_size):
    from tokenizers import Tokenizer
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import Whitespace
    words = ["<unk>", "<|im_start|>", "<|im_end|>", "system", "user", "assistant", "hello", "there"]
    words += [f"w{i}" for i in range(vocab_size - len(words))]
    tokenizer = Tokenizer(WordLevel({w: i for i, w in enumerate(words)}, unk_token="<unk>"))
    tokenizer.pre_tokenizer = Whitespace()
    tokenizer.save(str(folder / "tokenizer.json"))


@pytest.mark.gpu
def test_command_line_generates_from_ids_and_from_text(tmp_path):
    folder = make_folder("A", tmp_path)
    base = [sys.executable, str(ROOT / "bin" / "chat"), "--model_path", str(folder),
            "--model_type", "qwen3_fp32", "--max_new_tokens", "6", "--temperature", "0"]
    run = subprocess.run(base + ["--prompt_ids", "5,17,3"], capture_output=True, text=True,
                         timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert "Total Tokens:" in run.stdout and "tokens/sec" in run.stdout
    line = [l for l in run.stdout.split("\n") if l and l[0].isdigit()][0]
    ids = [int(x) for x in line.split()]
    assert 1 <= len(ids) <= 6
    # the same tokens as the Python entry point gives
    from edge_infer_amd.api import Model
    session = Model.from_pretrained(folder, "qwen3_fp32").new_session(capacity=64)
    assert session.generate([5, 17, 3], max_length=3 + 6, temperature=0.0) == ids
    # text in, text out, with a word-level tokenizer made for this test
    make_word_tokenizer(folder, 256)
    run = subprocess.run(base + ["--prompt", "hello there"], capture_output=True, text=True,
                         timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert "Total Tokens:" in run.stdout
    # chat loop: one turn, then quit
    run = subprocess.run(base, input="hello\nquit\n", capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    assert "Assistant:" in run.stdout and "Chat started" in run.stdout


def test_procedural_interface_without_a_model(capsys):
    """bindings/python/model_bridge.cpp:159-215: generating before init_model is an error;
    a failed init_model reports on stderr, returns False and leaves things as they were;
    only the GPU can be the default device."""
    from edge_infer_amd import api
    assert api._compat["session"] is None
    with pytest.raises(RuntimeError, match="Model not initialized"):
        api.generate_text_stream([1, 2, 3], lambda token: None)
    assert api.init_model({"architectures": ["NoSuchModel"]}, {}, "qwen3_bf16") is False
    assert "Error initializing model" in capsys.readouterr().err
    assert api.init_model({}, {}, "llama") is False          # a type this library does not have
    assert api._compat["session"] is None and api._compat["busy"] is False
    assert api.set_default_device("cpu") is False
    assert "Error setting default device" in capsys.readouterr().err
    assert api.get_default_device() == "cuda"
    assert api.is_cuda_available() == api.is_gpu_available()
    import inspect
    assert inspect.signature(api.generate_text_stream).parameters["top_k"].default == 50


def test_the_measurement_program_runs_on_one_gpu_only():
    """bench.py keeps its contract at one GPU; asked for more it says so in one line and
    exits with 2, before it touches any device."""
    root = Path(__file__).resolve().parent.parent
    done = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"],
                          capture_output=True, text=True, timeout=120)
    assert done.returncode == 2
    assert len(done.stdout.strip().splitlines()) == 1 and "one GPU" in done.stdout
