"""Command line in the manner of the reference's `main` (main.cpp:7-85): the same flag
names, defaults and meanings, the same interactive loop (lines until a blank line are one
prompt, end of input exits), errors as `[Fatal]: ...` with exit code 1.

Flags are parsed the gflags way: `--flag=value`, `--flag value`, `--flag` / `--noflag`
for booleans.  A prompt is text if the model folder has `tokenizer.json` (and the
`tokenizers` package is importable), otherwise token ids separated by spaces or commas.
"""
from __future__ import annotations

import os
import sys
from typing import Any, Dict, List, Tuple

# name -> (type, default, help); the first eight are the reference's (main.cpp:7-19)
FLAGS: Dict[str, Tuple[type, Any, str]] = {
    "model_path": (str, "", "Path to the model directory (required)"),
    "device": (int, 0, "GPU device ID"),
    "max_new_tokens": (int, 256, "Maximum number of tokens to generate"),
    "do_sample": (bool, True, "Whether to use sampling; if false, use greedy decoding"),
    "temperature": (float, 0.7, "Sampling temperature (higher = more creative)"),
    "top_k": (int, 50, "Sample from the top K most likely tokens (0 keeps all)"),
    "top_p": (float, 0.95, "Sample from the smallest set of tokens whose cumulative probability > p "
                           "(within the range [0, 1])"),
    "page_mode": (bool, False, "Whether to use PagedAttention (accepted; this engine is always paged)"),
    # this engine's own
    "dtype": (str, "bfloat16", "bfloat16 (serving) or float32 (true 32-bit path)"),
    "seed": (int, 0, "Seed of the sampling random numbers"),
    "prompt_ids": (str, "", "Token ids of one prompt (\"1,2,3\"): generate once and exit"),
    "prompt_ids_file": (str, "", "File with one prompt of token ids per line: generate for all of them and exit"),
    "random_weights": (bool, False, "Take only config.json from --model_path and fill the weights from --weights_seed"),
    "weights_seed": (int, 0, "Seed of the random weights"),
    "init_std": (float, 0.0, "Standard deviation of the random matrices (0: the configuration's initializer_range)"),
    "norm_std": (float, 0.0, "Standard deviation of the random norm weights around 1"),
    "stream": (bool, False, "Print the output as it is generated, not when the request has ended"),
    "ignore_eos": (bool, False, "Keep generating after the end-of-sequence token"),
    "kv_block_size": (int, 16, "Tokens per cache page"),
    "num_kv_blocks": (int, 0, "Cache pages (0: enough for max_num_seqs full-length requests)"),
    "max_num_seqs": (int, 8, "Most requests alive at once"),
    "max_num_batched_tokens": (int, 2048, "Token budget of one step"),
}


class FlagError(ValueError):
    pass


def _to_bool(text: str) -> bool:
    t = text.strip().lower()
    if t in ("1", "t", "true", "y", "yes"):
        return True
    if t in ("0", "f", "false", "n", "no"):
        return False
    raise FlagError(f"illegal value '{text}' for a boolean flag")


def parse_flags(argv: List[str]) -> Dict[str, Any]:
    values = {k: v[1] for k, v in FLAGS.items()}
    i = 0
    while i < len(argv):
        arg = argv[i]
        i += 1
        if not arg.startswith("-"):
            raise FlagError(f"unexpected argument '{arg}'")
        body = arg.lstrip("-")
        name, eq, val = body.partition("=")
        if name in ("help", "h"):
            raise FlagError(usage())
        if name not in FLAGS and name.startswith("no") and name[2:] in FLAGS and FLAGS[name[2:]][0] is bool and not eq:
            values[name[2:]] = False
            continue
        if name not in FLAGS:
            raise FlagError(f"unknown command line flag '{name}'")
        typ = FLAGS[name][0]
        if typ is bool:
            values[name] = _to_bool(val) if eq else True
            continue
        if not eq:
            if i >= len(argv):
                raise FlagError(f"flag '--{name}' is missing its argument")
            val = argv[i]
            i += 1
        try:
            values[name] = typ(val)
        except ValueError:
            raise FlagError(f"illegal value '{val}' specified for {typ.__name__} flag '{name}'") from None
    return values


def usage(prog: str = "tiny_llm") -> str:
    lines = [f"Usage: {prog} --model_path <path> [options]", ""]
    for name, (typ, default, text) in FLAGS.items():
        lines.append(f"    -{name} ({text}) type: {typ.__name__} default: {default!r}")
    return "\n".join(lines)


class _Text:
    """Text in and out through the model folder's tokenizer.json, or token ids as text."""

    def __init__(self, model_path: str):
        self.tok = None
        path = os.path.join(model_path, "tokenizer.json")
        if os.path.exists(path):
            try:
                from tokenizers import Tokenizer
                self.tok = Tokenizer.from_file(path)
            except Exception as e:  # noqa: BLE001
                print(f"[Warn]: tokenizer.json could not be loaded ({e}); prompts are token ids", file=sys.stderr)

    def encode(self, text: str) -> List[int]:
        if self.tok is not None:
            return list(self.tok.encode(text, add_special_tokens=True).ids)     # pipeline.cpp:113
        return parse_ids(text)

    def decode(self, ids: List[int]) -> str:
        if self.tok is not None:
            return self.tok.decode(ids, skip_special_tokens=True)              # pipeline.cpp:236
        return " ".join(str(i) for i in ids)


def parse_ids(text: str) -> List[int]:
    parts = text.replace(",", " ").split()
    try:
        return [int(p) for p in parts]
    except ValueError:
        raise FlagError("without tokenizer.json a prompt must be token ids separated by spaces or commas") from None


def _generate_streaming(engine, text: "_Text", prompt: List[int], params) -> List[int]:
    """Prints one prompt's output as it arrives: after every run of steps the text of all tokens so
    far is decoded again and what it gained is written (a token alone need not be whole characters)."""
    ids: List[int] = []
    shown = ""
    for _, fresh, _reason in engine.stream([prompt], params):
        ids += fresh
        now = text.decode(ids)
        if now.startswith(shown):
            sys.stdout.write(now[len(shown):])
        else:                                   # the tokenizer changed its mind about earlier text
            sys.stdout.write("\n" + now)
        sys.stdout.flush()
        shown = now
    sys.stdout.write("\n")
    sys.stdout.flush()
    return ids


def main(argv: List[str] = None) -> int:
    argv = sys.argv[1:] if argv is None else argv
    try:
        flags = parse_flags(argv)
    except FlagError as e:
        print(str(e), file=sys.stderr)
        return 1
    if not flags["model_path"]:
        print("Error: --model_path is mandatory.\n", file=sys.stderr)
        print(usage(), file=sys.stderr)
        return 1
    try:
        from . import Engine, EngineConfig, SamplingParams
        cfg = EngineConfig(dtype=flags["dtype"], kv_block_size=flags["kv_block_size"],
                           num_kv_blocks=flags["num_kv_blocks"] or None, max_num_seqs=flags["max_num_seqs"],
                           max_num_batched_tokens=flags["max_num_batched_tokens"], device=flags["device"],
                           seed=flags["seed"])
        if flags["random_weights"]:
            import json
            import os
            with open(os.path.join(flags["model_path"], "config.json")) as f:
                raw = json.load(f)
            engine = Engine(config=raw, engine_config=cfg, weights_seed=flags["weights_seed"],
                            init_std=flags["init_std"] or None, norm_std=flags["norm_std"])
        else:
            engine = Engine(flags["model_path"], engine_config=cfg)
        text = _Text(flags["model_path"])
        params = SamplingParams(max_new_tokens=flags["max_new_tokens"], do_sample=flags["do_sample"],
                                temperature=flags["temperature"], top_k=flags["top_k"], top_p=flags["top_p"],
                                ignore_eos=flags["ignore_eos"])
        if flags["prompt_ids"] or flags["prompt_ids_file"]:
            prompts = [parse_ids(flags["prompt_ids"])] if flags["prompt_ids"] else []
            if flags["prompt_ids_file"]:
                with open(flags["prompt_ids_file"]) as f:
                    prompts += [parse_ids(line) for line in f if line.strip()]
            if flags["stream"] and len(prompts) == 1:
                _generate_streaming(engine, text, prompts[0], params)
                return 0
            for out in engine.generate(prompts, params):
                print(text.decode(out))
            return 0
        print("\n>>> [Page Mode] Interactive Mode (Multi-line enabled) <<<")
        print(">>> Enter your prompt. Enter a blank line to end the current input. "
              "Enter EOF (Ctrl+D) to exit. <<<")
        while True:
            print("\n[Input] >", flush=True)
            buf, eof = "", True
            for line in sys.stdin:
                line = line.rstrip("\n")
                if line == "":
                    eof = False
                    break
                buf += line + "\n"
            if eof:
                break
            if not buf:
                print("The prompt is empty. Please re-enter.")
                continue
            if flags["stream"]:
                print("[Output] >", flush=True)
                _generate_streaming(engine, text, text.encode(buf), params)
                continue
            out = engine.generate([text.encode(buf)], params)[0]
            print("[Output] >\n" + text.decode(out), flush=True)
    except Exception as e:  # noqa: BLE001
        print(f"[Fatal]: {e}", file=sys.stderr)
        return 1
    print()
    return 0


if __name__ == "__main__":
    sys.exit(main())
