"""Command line in the manner of the reference's frontend/chat.py (names, meanings and
defaults of its options, frontend/chat.py:82-96):

    python -m edge_infer_amd.frontend.chat --model_path DIR --model_type qwen3_bf16 \\
        --max_new_tokens 424 --temperature 0.7 --top_p 1 --top_k 20

Without --prompt / --prompt_ids it is a chat loop (`quit` or `exit` ends it): the whole
conversation is rendered again for every turn, turns that exceed the session capacity are
refused, text is streamed as it becomes valid UTF-8, and time, tokens and tokens per
second are printed (frontend/chat.py:137-224).  With --prompt or --prompt_ids it generates
once and exits, which also serves folders that have no tokenizer (random weights).
The tokenizer is read from the folder's tokenizer.json with the `tokenizers` package;
nothing is ever downloaded.
"""
from __future__ import annotations

import argparse
import json
import sys
import time
from pathlib import Path

MODEL_TYPES = ("qwen3_bf16", "qwen3_fp32")


def load_tokenizer(model_path):
    path = Path(model_path) / "tokenizer.json"
    if not path.is_file():
        return None
    from tokenizers import Tokenizer
    return Tokenizer.from_file(str(path))


def render_chat(messages, model_path) -> str:
    """The folder's own chat template when it has one (tokenizer_config.json, rendered in a
    sandbox), else the ChatML layout that Qwen checkpoints use."""
    config_path = Path(model_path) / "tokenizer_config.json"
    if config_path.is_file():
        try:
            template = json.loads(config_path.read_text()).get("chat_template")
            if isinstance(template, str):
                from jinja2.sandbox import ImmutableSandboxedEnvironment
                env = ImmutableSandboxedEnvironment(trim_blocks=True, lstrip_blocks=True)
                return env.from_string(template).render(messages=messages,
                                                        add_generation_prompt=True)
        except Exception:  # an unusable template falls back to the plain layout
            pass
    text = "".join(f"<|im_start|>{m['role']}\n{m['content']}<|im_end|>\n" for m in messages)
    return text + "<|im_start|>assistant\n"


def _byte_alphabet():
    """The printable stand-in of every byte in byte-level vocabularies: bytes that print
    (33-126, 161-172, 174-255) stand for themselves, the others are numbered from 256 on in
    ascending order.  Returns stand-in character -> byte."""
    printable = [*range(33, 127), *range(161, 173), *range(174, 256)]
    table, extra = {}, 0
    for byte in range(256):
        if byte in printable:
            table[chr(byte)] = byte
        else:
            table[chr(256 + extra)] = byte
            extra += 1
    return table


def _whole_characters(data) -> int:
    """How many leading bytes of `data` can be decoded without cutting a UTF-8 character:
    if a lead byte among the last three announces more bytes than have arrived, the count
    stops before it."""
    size = len(data)
    for back in range(1, min(4, size) + 1):
        byte = data[size - back]
        if byte & 0xC0 == 0x80:
            continue                          # a continuation byte: look further back
        expected = 1 if byte < 0xC0 else 2 if byte < 0xE0 else 3 if byte < 0xF0 else 4
        return size if back >= expected else size - back
    return size


class TextStream:
    """Turns generated token ids into printable text piece by piece.

    Tokens of a byte-level vocabulary (the kind Qwen checkpoints have) are byte strings and
    a character may be spread over several tokens: their bytes are collected, and only the
    bytes that form whole characters are decoded and handed out; an unfinished tail waits for
    the next token.  For any other tokenizer the whole answer is decoded again at every token
    and what is new is handed out, except a tail of replacement characters, which the decoder
    writes for a character it cannot finish yet."""

    def __init__(self, tokenizer):
        self.tokenizer = tokenizer
        self.text = ""                      # everything handed out so far
        self._bytes = bytearray()           # byte-level: bytes not handed out yet
        self._ids = []                      # otherwise: every token so far
        self._alphabet = self._special = None
        describe = getattr(tokenizer, "to_str", None)
        if describe is not None:
            decoder = json.loads(describe()).get("decoder") or {}
            stages = decoder.get("decoders", [decoder])
            if any(stage.get("type") == "ByteLevel" for stage in stages):
                self._alphabet = _byte_alphabet()
                self._special = {index: token.content for index, token
                                 in tokenizer.get_added_tokens_decoder().items()}

    def push(self, token: int) -> str:
        """The text that this token completes (possibly empty)."""
        if self._alphabet is None:
            self._ids.append(token)
            decoded = self.tokenizer.decode(self._ids, skip_special_tokens=True)
            settled = decoded.rstrip("\ufffd")
            if len(decoded) - len(settled) > 3:      # more than one character can lack: real ones
                settled = decoded
            if not settled.startswith(self.text):    # the decoder changed its mind: keep what is out
                return ""
            piece = settled[len(self.text):]
        else:
            if token in self._special:
                return ""                            # markers of the chat layout are not text
            symbol = self.tokenizer.id_to_token(token) or ""
            try:
                self._bytes += bytes(self._alphabet[char] for char in symbol)
            except KeyError:                         # an added plain-text token
                self._bytes += symbol.encode("utf-8")
            whole = _whole_characters(self._bytes)
            piece = bytes(self._bytes[:whole]).decode("utf-8", errors="replace")
            del self._bytes[:whole]
        self.text += piece
        return piece

    def finish(self) -> str:
        """What was still held back when generation ended."""
        if self._alphabet is None:
            decoded = self.tokenizer.decode(self._ids, skip_special_tokens=True) if self._ids else ""
            piece = decoded[len(self.text):] if decoded.startswith(self.text) else ""
        else:
            piece = bytes(self._bytes).decode("utf-8", errors="replace")
            self._bytes.clear()
        self.text += piece
        return piece


def build_parser() -> argparse.ArgumentParser:
    parser = argparse.ArgumentParser(description="Qwen3 chat / generation on one MI355X")
    parser.add_argument("--model_path", type=str, required=True,
                        help="local folder with config.json, safetensors and (for text) tokenizer.json")
    parser.add_argument("--model_type", type=str, default="qwen3_bf16", choices=MODEL_TYPES,
                        help="qwen3_bf16, or qwen3_fp32 for the true 32-bit path")
    parser.add_argument("--device", type=str, default="cuda", choices=["cuda"],
                        help="execution device (this library runs on the GPU only)")
    parser.add_argument("--system_prompt", type=str, default="You are a helpful AI assistant.")
    parser.add_argument("--max_new_tokens", "--max_length", dest="max_new_tokens", type=int,
                        default=424, help="maximum generated token count")
    parser.add_argument("--context_capacity", type=int, default=None,
                        help="session token capacity (default: min(4096, model limit))")
    parser.add_argument("--temperature", type=float, default=0.7)
    parser.add_argument("--top_p", type=float, default=1.0)
    parser.add_argument("--top_k", type=int, default=20)
    parser.add_argument("--seed", type=int, default=None,
                        help="sampler seed (default: taken from the clock)")
    parser.add_argument("--prompt", type=str, default=None,
                        help="generate once for this user message and exit")
    parser.add_argument("--prompt_ids", type=str, default=None,
                        help="generate once for these comma-separated token ids and exit")
    return parser


def generate_once(session, input_ids, args, tokenizer, out=sys.stdout):
    """Stream one answer; returns (token ids, seconds from the first token, text)."""
    max_length = min(session.capacity, len(input_ids) + args.max_new_tokens)
    tokens, started = [], [None]
    stream = TextStream(tokenizer) if tokenizer is not None else None

    def on_token(token):
        if started[0] is None:
            started[0] = time.monotonic()
        tokens.append(token)
        piece = f"{token} " if stream is None else stream.push(token)
        if piece:
            print(piece, end="", file=out, flush=True)

    session.generate(input_ids, on_token, max_length=max_length, temperature=args.temperature,
                     top_p=args.top_p, top_k=args.top_k)
    elapsed = time.monotonic() - started[0] if started[0] is not None else 0.0
    if stream is None:
        return tokens, elapsed, ""
    rest = stream.finish()
    if rest:
        print(rest, end="", file=out, flush=True)
    return tokens, elapsed, stream.text


def report(tokens, elapsed, out=sys.stdout):
    speed = len(tokens) / elapsed if elapsed > 0 else 0.0
    print("\n", file=out)
    print(f"Total Time: {elapsed:.2f} seconds", file=out)
    print(f"Total Tokens: {len(tokens)}", file=out)
    print(f"Average Speed: {speed:.2f} tokens/sec\n", file=out)


def main(argv=None) -> int:
    parser = build_parser()
    args = parser.parse_args(argv)
    if args.max_new_tokens <= 0:
        parser.error("--max_new_tokens must be positive")

    from ..api import Model
    model = Model.from_pretrained(args.model_path, args.model_type, device=args.device)
    cfg = model.config
    print(f"Model Type: {args.model_type}")
    print(f"Hidden Size: {cfg.hidden_size}")
    print(f"Num Layers: {cfg.num_hidden_layers}")
    print(f"Num Attention Heads: {cfg.num_attention_heads}")
    print(f"Num KV Heads: {cfg.num_key_value_heads}")
    print(f"Head Dimension: {cfg.head_dim}")
    seed = args.seed if args.seed is not None else time.time_ns() & 0xFFFFFFFF
    session = model.new_session(capacity=args.context_capacity, seed=seed)
    print(f"Model initialized on {model.device}; context capacity: {session.capacity} tokens.\n")
    tokenizer = load_tokenizer(args.model_path)

    if args.prompt_ids is not None:
        ids = [int(piece) for piece in args.prompt_ids.replace(",", " ").split()]
        tokens, elapsed, _ = generate_once(session, ids, args, tokenizer)
        report(tokens, elapsed)
        return 0
    if tokenizer is None:
        parser.error(f"{args.model_path} has no tokenizer.json: use --prompt_ids")

    messages = [{"role": "system", "content": args.system_prompt}]
    if args.prompt is not None:
        messages.append({"role": "user", "content": args.prompt})
        ids = tokenizer.encode(render_chat(messages, args.model_path), add_special_tokens=False).ids
        if len(ids) >= session.capacity:
            parser.error("the prompt exceeds the session capacity")
        tokens, elapsed, _ = generate_once(session, ids, args, tokenizer)
        report(tokens, elapsed)
        return 0

    print("Chat started. Type 'quit' or 'exit' to quit.\n")
    while True:
        try:
            user_message = input("User: ").strip()
        except EOFError:
            break
        if user_message.lower() in {"quit", "exit"}:
            break
        if not user_message:
            continue
        messages.append({"role": "user", "content": user_message})
        ids = tokenizer.encode(render_chat(messages, args.model_path), add_special_tokens=False).ids
        if len(ids) >= session.capacity:
            messages.pop()
            print("Conversation exceeds the session capacity. Start a new chat or use a "
                  "larger capacity.")
            continue
        print("Assistant: ", end="", flush=True)
        try:
            tokens, elapsed, text = generate_once(session, ids, args, tokenizer)
        except Exception as error:  # the turn is dropped, the chat goes on
            messages.pop()
            print(f"\nGeneration failed: {error}", file=sys.stderr)
            continue
        messages.append({"role": "assistant", "content": text})
        report(tokens, elapsed)
    return 0


if __name__ == "__main__":
    sys.exit(main())
