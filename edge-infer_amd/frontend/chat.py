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


def decode_stream_incremental(tokenizer, token_ids, rendered_text):
    """(new text that is safe to print, text rendered so far): text that ends inside a
    multi-byte character is held back until the character is complete."""
    decoded = tokenizer.decode(token_ids, skip_special_tokens=True)
    prefix = 0
    limit = min(len(rendered_text), len(decoded))
    while prefix < limit and rendered_text[prefix] == decoded[prefix]:
        prefix += 1
    pending = decoded[prefix:]
    broken = pending.find("�")
    if broken != -1:
        safe = pending[:broken]
        return safe, decoded[:prefix + len(safe)]
    return pending, decoded


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
    tokens, rendered, started = [], "", [None]

    def on_token(token):
        if started[0] is None:
            started[0] = time.monotonic()
        tokens.append(token)
        if tokenizer is None:
            print(token, end=" ", file=out, flush=True)
            return
        nonlocal rendered
        piece, rendered = decode_stream_incremental(tokenizer, tokens, rendered)
        if piece:
            print(piece, end="", file=out, flush=True)

    session.generate(input_ids, on_token, max_length=max_length, temperature=args.temperature,
                     top_p=args.top_p, top_k=args.top_k)
    elapsed = time.monotonic() - started[0] if started[0] is not None else 0.0
    text = tokenizer.decode(tokens, skip_special_tokens=True) if tokenizer is not None else ""
    if tokenizer is not None and text[len(rendered):]:
        print(text[len(rendered):], end="", file=out, flush=True)
    return tokens, elapsed, text


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
