"""Complete prompts with a local model, on the command line.

The options are those of the reference's scripts/complete.py (:45-59): --model,
--max-new-tokens, --temperature (<= 0: greedy), --top-p, --device; so are the commands of its
prompt loop (/clear, /history, /exit, /quit; :156-180). This one runs the framework's own
engine. Prompts are token ids (``--tokens 15496,11,995`` or a line of numbers); text works when
the model folder has a tokenizer.json."""

from __future__ import annotations

import argparse
import sys
from pathlib import Path


def parse_args(argv=None) -> argparse.Namespace:
    parser = argparse.ArgumentParser(description="Complete prompts with the local model")
    parser.add_argument("--model", default="models/gpt2", help="Model directory")
    parser.add_argument("--max-new-tokens", type=int, default=64)
    parser.add_argument("--temperature", type=float, default=0.8)
    parser.add_argument("--top-p", type=float, default=0.95)
    parser.add_argument("--device", default="auto", choices=("auto", "cpu", "cuda"), help="Inference device")
    parser.add_argument("--dtype", default="bfloat16", choices=("bfloat16", "float32"))
    parser.add_argument("--seed", type=int, default=0, help="Seed of the sampler")
    parser.add_argument("--tokens", default=None, help="Prompt as comma-separated token ids; prints the continuation and exits")
    return parser.parse_args(argv)


def load_tokenizer(model_dir):
    path = Path(model_dir) / "tokenizer.json"
    if not path.is_file():
        return None
    try:
        from tokenizers import Tokenizer
    except ImportError:
        return None
    return Tokenizer.from_file(str(path))


def parse_ids(text: str) -> list[int] | None:
    parts = text.replace(",", " ").split()
    try:
        return [int(p) for p in parts] if parts else None
    except ValueError:
        return None


def main(argv=None) -> int:
    args = parse_args(argv)
    if args.device == "cpu":
        print("this engine runs on the GPU only: there is no CPU path", file=sys.stderr)
        return 2
    from ..engine.engine import Engine, EngineOptions

    engine = Engine(args.model, EngineOptions(dtype=args.dtype, max_sessions=4))
    tokenizer = load_tokenizer(args.model)
    eos = engine.config.eos_token_id

    def complete(ids: list[int], turn: int) -> list[int]:
        return engine.generate([ids], max_new_tokens=args.max_new_tokens, temperature=max(args.temperature, 0.0),
                               top_p=args.top_p, seed=args.seed + turn, eos_token_id=eos)[0]

    if args.tokens is not None:
        ids = parse_ids(args.tokens)
        if ids is None:
            print("--tokens needs comma-separated integers", file=sys.stderr)
            return 2
        print(",".join(str(t) for t in complete(ids, 0)))
        return 0

    history: list[tuple[str, str]] = []
    print("Enter a prompt (token ids, or text if the folder has a tokenizer). /clear /history /exit", file=sys.stderr)
    turn = 0
    while True:
        try:
            line = input("> ").strip()
        except (EOFError, KeyboardInterrupt):
            break
        if not line:
            continue
        if line in ("/exit", "/quit"):
            break
        if line == "/clear":
            history.clear()
            continue
        if line == "/history":
            for prompt, completion in history:
                print(f"> {prompt}\n{completion}")
            continue
        ids = parse_ids(line)
        as_text = ids is None
        if as_text:
            if tokenizer is None:
                print("no tokenizer.json in the model folder: enter token ids", file=sys.stderr)
                continue
            ids = tokenizer.encode(line).ids
        try:
            new = complete(ids, turn)
        except Exception as error:
            print(f"error: {error}", file=sys.stderr)
            continue
        turn += 1
        completion = tokenizer.decode(new) if as_text else " ".join(str(t) for t in new)
        history.append((line, completion))
        print(completion)
    return 0


if __name__ == "__main__":
    sys.exit(main())
