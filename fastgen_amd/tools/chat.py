"""``fgchat``: the reference's command line (``fastgen/tools/chat.py:87-216``)
with its option names, generating in-process.  Without a prompt option it is
the reference's dialogue loop (needs a tokenizer in the model folder; ``/q``
quits, ``/r`` drops the last exchange); with one it generates once and exits:

    fgchat MODEL --prompt-ids 1,2,3 --max-tokens 32 --temperature 0
    fgchat MODEL --random-prompt 128 --max-tokens 64
    fgchat --config config.json --random-weights 2 --random-prompt 128 --max-tokens 64 --num-pages 16

``--random-weights SEED`` needs no weights on disk: the configuration comes from ``--config FILE`` (or from
``config.json`` in MODEL) and the tensors are drawn on the GPU from the seed.
"""

from __future__ import annotations

import argparse
import logging
import queue
import sys
import time
from typing import List, Optional

import torch


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="fgchat", description="Generate with a model folder on one MI355X.")
    ap.add_argument("model", nargs="?", default=None,
                    help="model folder (config.json, safetensors, optionally tokenizer.json)")
    ap.add_argument("--temperature", type=float, default=0.7, help="0 is greedy (default 0.7)")
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--max-tokens", type=int, default=None, help="most tokens to generate")
    ap.add_argument("--gpu-gb", type=float, default=20, help="memory budget for weights and cache")
    ap.add_argument("--tensor-parallel", type=int, default=1, help="accepted for compatibility; must be 1")
    ap.add_argument("--verbose", action="store_true")
    # beyond the reference: generate once without a dialogue
    ap.add_argument("--prompt", help="text prompt (needs tokenizer.json in the model folder)")
    ap.add_argument("--prompt-ids", help="comma-separated token ids")
    ap.add_argument("--random-prompt", type=int, metavar="LEN", help="a prompt of LEN uniform random ids")
    ap.add_argument("--seed", type=int, default=777)
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--page-size", type=int, default=64)
    ap.add_argument("--max-seq", type=int, default=-1, help="cache size in tokens (default: from --gpu-gb)")
    ap.add_argument("--max-step-tokens", type=int, default=8192, help="token budget of one step")
    ap.add_argument("--num-pages", type=int, default=None, help="cache size in pages (overrides --max-seq and --gpu-gb)")
    ap.add_argument("--random-weights", type=int, default=None, metavar="SEED",
                    help="no weights are read: they are drawn on the GPU from this seed")
    ap.add_argument("--config", default=None, metavar="FILE",
                    help="a config.json for --random-weights (default: the one in MODEL)")
    ap.add_argument("--drop-stop-token", action="store_true",
                    help="a stop id that ends the generation is not printed among the ids")
    return ap


def main(argv: Optional[List[str]] = None) -> int:
    import json

    from ..engine import Model
    from ..generate import Fastgen, GenArgs, Packet, memory_budget
    from .tokenizer import FolderTokenizer

    a = build_parser().parse_args(argv)
    if a.tensor_parallel != 1:
        print("fgchat: this engine runs on one GPU; --tensor-parallel must be 1", file=sys.stderr)
        return 2
    if a.model is None and (a.random_weights is None or a.config is None):
        print("fgchat: give a model folder, or --random-weights SEED with --config FILE", file=sys.stderr)
        return 2
    if a.config is not None and a.random_weights is None:
        print("fgchat: --config is for --random-weights; a model folder brings its own config.json", file=sys.stderr)
        return 2
    logging.basicConfig(level=logging.INFO if a.verbose else logging.WARNING)
    tokenizer = FolderTokenizer.maybe(a.model) if a.model is not None else None
    gen_args = GenArgs(
        use_sampling=bool(a.temperature), temperature=a.temperature, top_p=a.top_p, max_batch=1,
        max_gen=a.max_tokens, gpu_gb=a.gpu_gb, cache_block=a.page_size, max_seq=a.max_seq,
        max_prefill=a.max_step_tokens, seed=a.seed, dtype=getattr(torch, a.dtype),
    )
    stop_tokens = tokenizer.stop_tokens if tokenizer else None
    if a.random_weights is not None:
        from ..config import read_config_json

        if a.config is not None:
            with open(a.config) as f:
                config = json.load(f)
        else:
            config = read_config_json(a.model)
        budget = memory_budget(gen_args) if a.num_pages is None else None
        model = Model.random(config, a.random_weights, gen_args.dtype, "cuda:0", memory_budget=budget)
        fg = Fastgen.from_model(model, gen_args, stop_tokens if stop_tokens is not None else (), a.num_pages)
    elif a.num_pages is not None:
        fg = Fastgen.from_model(Model.from_folder(a.model, gen_args.dtype, "cuda:0"), gen_args, stop_tokens, a.num_pages)
    else:
        fg = Fastgen.build(a.model, gen_args, stop_tokens=stop_tokens)
    q: "queue.Queue" = queue.Queue()
    gen = fg.generate(q)

    def run(tokens: List[int]) -> List[int]:
        t0 = time.time()
        q.put(Packet(thread_id=0, tokens=tokens))
        pkt = next(gen)
        dt = time.time() - t0
        print(f"[{len(pkt.tokens)} tokens, {len(pkt.tokens) / dt:.1f} tok/s]", file=sys.stderr)
        return pkt.tokens

    one_shot = a.prompt is not None or a.prompt_ids is not None or a.random_prompt is not None
    if one_shot:
        if a.prompt is not None:
            if tokenizer is None:
                print("fgchat: --prompt needs tokenizer.json in the model folder", file=sys.stderr)
                return 2
            ids = tokenizer.encode_dialog([{"role": "user", "content": a.prompt}])
        elif a.prompt_ids is not None:
            ids = [int(x) for x in a.prompt_ids.replace(" ", "").split(",") if x]
        else:
            g = torch.Generator().manual_seed(a.seed)
            ids = torch.randint(0, fg.engine.model.vocab_size, (a.random_prompt,), generator=g).tolist()
        out = run(ids)
        if a.drop_stop_token and out and out[-1] in fg.stop_tokens:
            out = out[:-1]
        print(",".join(str(t) for t in out))
        if tokenizer is not None:
            print(tokenizer.decode([t for t in out if t not in tokenizer.stop_tokens]))
        return 0
    if tokenizer is None:
        print("fgchat: a dialogue needs tokenizer.json in the model folder; use --prompt-ids or --random-prompt",
              file=sys.stderr)
        return 2
    print("Commands: /r <N> go back to before round N; /m a message of several lines, ended by a line"
          " that holds only '.'; /q quit", file=sys.stderr)
    return dialogue_loop(tokenizer, run)


def read_turn(dialog: List[dict], read=input) -> Optional[str]:
    """One turn of the dialogue's prompt (``fastgen/tools/chat.py:170-195``): returns the user's message, or
    None when the loop should ask again (a command was carried out); raises EOFError to quit.  ``/r <N>`` cuts
    the dialogue back to before round N (a round is a user message and its answer), ``/r`` alone drops the last
    round; ``/m`` reads lines until one that is a single '.'; ``/q`` quits."""
    n_round = 1 + len(dialog) // 2
    line = read(f"{n_round}> ").strip()
    word, _, rest = line.partition(" ")
    if word == "/q":
        raise EOFError
    if word == "/r":
        try:
            n = int(rest) if rest.strip() else n_round - 1
            if n < 1:
                raise ValueError
            del dialog[2 * (n - 1):]
        except ValueError:
            print("invalid command", file=sys.stderr)
        return None
    if word == "/m" and not rest.strip():
        lines: List[str] = []
        while True:
            more = read(f"{n_round}>> ")
            if more.strip() == ".":
                break
            lines.append(more)
        return "\n".join(lines)
    return line


def dialogue_loop(tokenizer, run, read=input, write=print) -> int:
    dialog: List[dict] = []
    while True:
        try:
            msg = read_turn(dialog, read)
        except EOFError:
            return 0
        if msg is None:
            continue
        dialog.append({"role": "user", "content": msg})
        out = run(tokenizer.encode_dialog(dialog))
        if out and out[-1] in tokenizer.stop_tokens:
            out = out[:-1]  # tools/chat.py:205-206
        text = tokenizer.decode(out)
        write(text)
        dialog.append({"role": "assistant", "content": text})


if __name__ == "__main__":
    sys.exit(main())
