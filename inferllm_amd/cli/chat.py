"""Command line in the manner of the reference's `chat` (application/chat.cpp:20-104).

Options the reference has keep their names and meanings: -m/--model, -s/--seed,
-t/--threads, --top_k, --top_p, --temp, --repeat_last_n, --repeat_penalty,
-c/--ctx_size, -d/--dtype, -g, --type, --mmap, -h/--help, with the reference's
defaults (top_k 40, top_p 0.95, temp 0.10, repeat_penalty 1.10, repeat_last_n 64,
ctx_size 2048, seed -1 = from the clock).  Differences: the model is a folder
(config.json + safetensors), dtype is float32 or bfloat16, the device is a GPU,
`--temp 0` is greedy, an unknown option prints the usage and exits with 2 (the
reference exits 0 silently, chat.cpp:98-100), and `-n/--n_predict` is honoured
(the reference declares it and never reads it, chat.cpp:23).

Prompts are token ids (`--prompt-ids "1,5,9"`, or `--prompt-ids-file` with one
request per line: the lines form a batch), or text (`-p/--prompt`) when the model
folder has a tokenizer.json or a tokenizer.model.  Without a prompt the program reads the
turns of one conversation from standard input, one per line, like the reference's interactive
loop (chat.cpp:221-275): every turn goes on from what was said before, until the
context is full or the input ends.
"""
from __future__ import annotations

import argparse
import os
import sys
import time
from typing import List, Optional


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="chat", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("-m", "--model", help="model folder (config.json and model.safetensors)")
    ap.add_argument("-s", "--seed", type=int, default=-1, help="RNG seed (default: -1, from the clock)")
    ap.add_argument("-t", "--threads", type=int, default=1,
                    help="accepted for compatibility; computing is on the GPU")
    ap.add_argument("--top_k", type=int, default=40, help="top-k sampling (default: 40; 0 = off)")
    ap.add_argument("--top_p", type=float, default=0.95, help="top-p sampling (default: 0.95; 1 = off)")
    ap.add_argument("--temp", type=float, default=0.10, help="temperature (default: 0.1; 0 = greedy)")
    ap.add_argument("--repeat_last_n", type=int, default=64,
                    help="last n tokens to consider for penalize (default: 64)")
    ap.add_argument("--repeat_penalty", type=float, default=1.10,
                    help="penalize repeat sequence of tokens (default: 1.1; 1 = off)")
    ap.add_argument("-c", "--ctx_size", type=int, default=2048, help="size of the context (default: 2048)")
    ap.add_argument("-d", "--dtype", default="bfloat16", choices=["float32", "bfloat16"],
                    help="compute type (default: bfloat16)")
    ap.add_argument("-g", dest="device", default="GPU", help="compute device type: GPU (CPU is refused)")
    ap.add_argument("--type", dest="mtype", default=None,
                    help="model type name; must agree with config.json if given (llama, llama2)")
    ap.add_argument("--mmap", action="store_true",
                    help="accepted for compatibility; safetensors files are always memory-mapped")
    ap.add_argument("-n", "--n_predict", type=int, default=128, help="new tokens to predict (default: 128)")
    ap.add_argument("-p", "--prompt", default=None, help="text prompt (needs tokenizer.json or tokenizer.model in the model folder)")
    ap.add_argument("--prompt-ids", default=None, help='prompt as token ids, e.g. "1,5,9"')
    ap.add_argument("--prompt-ids-file", default=None, help="file with one request (token ids) per line")
    ap.add_argument("--stop-ids", default=None, help="stop token ids (default: the model's eos ids)")
    ap.add_argument("--max-batch", type=int, default=8, help="most sequences decoded together (default: 8)")
    ap.add_argument("--random", dest="random_config", default=None,
                    help="config.json to build random weights from instead of --model")
    ap.add_argument("--weights-seed", type=int, default=0, help="seed of --random weights")
    ap.add_argument("--summary", action="store_true", help="print prefill and decode token/s at the end")
    ap.add_argument("--profile", action="store_true",
                    help="time every kernel call with HIP events (steps run without HIP graphs) and "
                         "print a table per op at the end")
    return ap


def parse_ids(text: str) -> List[int]:
    ids = [int(t) for t in text.replace(",", " ").split()]
    if not ids:
        raise ValueError("empty list of token ids")
    return ids


class _Text:
    """Text in and out through the folder's tokenizer.json or, without one, its tokenizer.model
    (a SentencePiece model, as LLaMA-2 checkpoints bring it), if there is either."""

    def __init__(self, model_dir: Optional[str]):
        self.tok = self.pieces = None
        path = os.path.join(model_dir, "tokenizer.json") if model_dir else None
        spm = os.path.join(model_dir, "tokenizer.model") if model_dir else None
        if path and os.path.isfile(path):
            from tokenizers import Tokenizer
            self.tok = Tokenizer.from_file(path)
        elif spm and os.path.isfile(spm):
            from sentencepiece import SentencePieceProcessor
            self.pieces = SentencePieceProcessor(model_file=spm)

    @property
    def known(self) -> bool:
        """Whether the folder brought a tokenizer (else ids are shown as numbers)."""
        return self.tok is not None or self.pieces is not None

    def encode(self, text: str, bos: Optional[int]) -> List[int]:
        if self.tok is not None:
            ids = self.tok.encode(text, add_special_tokens=False).ids
        elif self.pieces is not None:
            ids = list(self.pieces.encode(text))
        else:
            raise SystemExit("text prompts need a tokenizer.json or a tokenizer.model in the model "
                             "folder; use --prompt-ids")
        return ([bos] if bos is not None else []) + ids      # the reference prepends BOS (model_imp.cpp:123-125)

    def show(self, ids: List[int]) -> str:
        if self.tok is not None:
            return self.tok.decode(ids)
        if self.pieces is not None:
            return self.pieces.decode(list(ids))
        return " ".join(str(i) for i in ids)

    def printer(self):
        """`put(token)` prints an answer as its tokens come (the reference prints every token as it
        is generated, application/chat.cpp:232-236): ids as numbers, text as what the answer so
        far decodes to beyond what is already out (a token that ends inside a character waits
        for the rest of it)."""
        ids: List[int] = []
        out = [""]

        def put(token: int) -> None:
            if not self.known:
                print(token, end=" ", flush=True)
                return
            ids.append(token)
            now = self.show(ids)
            if now.endswith("\ufffd"):
                return
            print(now[len(os.path.commonprefix([out[0], now])):], end="", flush=True)
            out[0] = now
        return put


def main(argv=None) -> int:
    ap = build_parser()
    try:
        args = ap.parse_args(argv)
    except SystemExit as e:
        return int(e.code or 0) if e.code in (0, None) else 2
    if args.device.upper() != "GPU":
        print(f"chat: device type {args.device!r} is not served: this engine computes on a GPU only",
              file=sys.stderr)
        return 2
    if not args.model and not args.random_config:
        ap.print_usage(sys.stderr)
        print("chat: -m/--model (or --random CONFIG) is required", file=sys.stderr)
        return 2

    import json

    from .. import Engine
    from ..config import config_from_dict

    seed = args.seed if args.seed >= 0 else int(time.time())
    kw = dict(dtype=args.dtype, max_batch=args.max_batch, max_seq_len=args.ctx_size,
              use_graphs=not args.profile)
    if args.random_config:
        with open(args.random_config, "r", encoding="utf-8") as f:
            config = config_from_dict(json.load(f))
        eng = Engine.from_random(config, seed=args.weights_seed, **kw)
    else:
        eng = Engine.from_pretrained(args.model, **kw)
    if args.mtype is not None:
        family = tuple(getattr(type(eng.config), "cli_type_names", ()))
        if args.mtype not in family:
            print(f"chat: --type {args.mtype!r} does not fit the model's architecture "
                  f"{eng.spec.architecture!r}", file=sys.stderr)
            return 2
    text = _Text(args.model)
    stops = parse_ids(args.stop_ids) if args.stop_ids else None

    def run(prompts: List[List[int]]) -> None:
        stream = len(prompts) == 1                        # one request: printed as it comes
        put = text.printer()

        def show(i: int, tok: int) -> None:
            put(tok)
        # the decode graph of this batch is captured before the request starts, so that its first
        # decoded tokens do not wait for the capture; no throwaway prompt is run: for a one-shot
        # command that would be the whole prompt twice, and `--summary` shows what the user waited
        eng.warm_up([min(len(prompts), args.max_batch)], max(len(p) for p in prompts) + args.n_predict)
        outs = eng.generate(prompts, temperature=args.temp, top_k=args.top_k, top_p=args.top_p,
                            repeat_penalty=args.repeat_penalty, repeat_last_n=args.repeat_last_n,
                            seed=seed, max_new_tokens=args.n_predict, stop_token_ids=stops,
                            on_token=show if stream else None)
        if stream:
            print(flush=True)
        else:
            for o in outs:
                print(text.show(o), flush=True)
        if args.summary:
            print(eng.last_stats.summary(), file=sys.stderr, flush=True)

    if args.profile:
        from ..kernels.profile import kernel_timing
        timing = kernel_timing()
        times = timing.__enter__()
        import atexit
        atexit.register(lambda: (print(times.table(), file=sys.stderr, flush=True),
                                 timing.__exit__(None, None, None)))

    prompts: List[List[int]] = []
    if args.prompt_ids:
        prompts.append(parse_ids(args.prompt_ids))
    if args.prompt_ids_file:
        with open(args.prompt_ids_file, "r", encoding="utf-8") as f:
            prompts.extend(parse_ids(line) for line in f if line.strip())
    if args.prompt is not None:
        prompts.append(text.encode(args.prompt, eng.spec.bos_token_id))
    if prompts:
        run(prompts)
        return 0
    # No prompt: turns from standard input, one a line, in ONE context that goes on from turn to
    # turn until it is full or the input ends, like the reference's loop (chat.cpp:221-275).
    with eng.session(temperature=args.temp, top_k=args.top_k, top_p=args.top_p,
                     repeat_penalty=args.repeat_penalty, repeat_last_n=args.repeat_last_n,
                     seed=seed, stop_token_ids=stops) as talk:
        eng.warm_up([1], args.ctx_size)
        first = True
        for line in sys.stdin:
            line = line.strip()
            if not line:
                continue
            try:
                ids = parse_ids(line)
            except ValueError:
                ids = text.encode(line, eng.spec.bos_token_id if first else None)
            if len(ids) + 1 > talk.remaining:
                print(f"chat: the context is full ({talk.remaining} tokens left)", file=sys.stderr)
                break
            first = False
            talk.say(ids, args.n_predict, on_token=text.printer())
            print(flush=True)
            if args.summary:
                print(talk.last_stats.summary(), file=sys.stderr, flush=True)
            if talk.remaining <= 0:
                break
    return 0


if __name__ == "__main__":
    sys.exit(main())
