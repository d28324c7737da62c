"""Python front in the manner of scripts/run_prompt.py of the reference: turn a
text prompt into token ids with the model folder's tokenizer (chat template,
thinking off), run the engine, decode the new ids.  The reference shells out
to its binary and parses the `New token ids:` line (scripts/run_prompt.py:9-27,
:122-145); `--engine` does the same here with this package's command line,
and without it the engine is called in-process."""
from __future__ import annotations

import argparse
import re
import subprocess
import sys
from typing import List

from .cli import templated_prompt
from .token_ids import parse_token_ids

# the output contract of the command line: the line "New token ids:", then a line with the ids
_NEW_IDS = re.compile(r"^[ \t]*New token ids:[ \t]*\r?\n([^\r\n]*)", re.MULTILINE)


def parse_new_token_ids(output: str) -> List[int]:
    """The ids that the command line printed after `New token ids:` (`<none>`: no ids)."""
    found = _NEW_IDS.search(output)
    if found is None:
        raise RuntimeError("the engine's output holds no 'New token ids:' line with ids after it")
    ids = found.group(1).strip()
    if ids == "<none>":
        return []
    try:
        return parse_token_ids(ids)
    except ValueError as e:
        raise RuntimeError(f"the line after 'New token ids:' is no id list: {e}") from None


def encode_prompt(tokenizer, model_dir: str, prompt: str, use_chat_template: bool) -> List[int]:
    text = templated_prompt(model_dir, prompt, enable_thinking=False) if use_chat_template else prompt
    return list(tokenizer.encode(text, add_special_tokens=False).ids)


def options(argv=None) -> argparse.Namespace:
    """The reference's option names (scripts/run_prompt.py:96-121) and this front's own --dtype."""
    p = argparse.ArgumentParser(prog="run_prompt", description="Tokenize a prompt, generate greedily, print the reply.")
    p.add_argument("--model", required=True, help="model folder with tokenizer.json")
    p.add_argument("--engine", default=None, help="the command line to run as a child process (default: in-process)")
    p.add_argument("--prompt", required=True)
    p.add_argument("--max-tokens", type=int, default=64)
    p.add_argument("--device", default="cuda")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--eos-token-id", type=int, default=None, help="default: the id of the tokenizer's <|im_end|>")
    p.add_argument("--no-chat-template", action="store_true")
    p.add_argument("--show-full-text", action="store_true")
    return p.parse_args(argv)


def generate_in_child(engine: str, args: argparse.Namespace, ids_text: str, eos) -> "tuple[int, List[int]]":
    """Greedy generation by the command line `engine` as a child process: (its exit code, the new
    ids read from the `New token ids:` line of what it printed, which is echoed)."""
    child_args = {"--model": args.model, "--input-ids": ids_text, "--max-tokens": str(args.max_tokens),
                  "--device": args.device, "--temperature": "0", "--dtype": args.dtype}
    if eos is not None:
        child_args["--eos-token-id"] = str(eos)
    child = subprocess.run([engine] + [x for pair in child_args.items() for x in pair], text=True,
                           stdout=subprocess.PIPE, stderr=subprocess.STDOUT, check=False)
    sys.stdout.write("--- output of " + engine + " ---\n" + child.stdout + "--- end of its output ---\n")
    if child.returncode != 0:
        return child.returncode, []
    return 0, parse_new_token_ids(child.stdout)


def main(argv=None) -> int:
    import os

    from tokenizers import Tokenizer

    args = options(argv)
    tokenizer = Tokenizer.from_file(os.path.join(args.model, "tokenizer.json"))
    eos = tokenizer.token_to_id("<|im_end|>") if args.eos_token_id is None else args.eos_token_id
    prompt_ids = encode_prompt(tokenizer, args.model, args.prompt, not args.no_chat_template)
    ids_text = ",".join(str(i) for i in prompt_ids)
    print(f"prompt: {len(prompt_ids)} tokens\n  {ids_text}\n")

    if args.engine is None:
        from .generate import generate

        new_ids = generate(args.model, [prompt_ids], args.max_tokens, 0.0, -1 if eos is None else eos,
                           args.dtype, args.device)[0]
    else:
        code, new_ids = generate_in_child(args.engine, args, ids_text, eos)
        if code != 0:
            return code
    print(f"reply: {len(new_ids)} tokens")
    print(tokenizer.decode(new_ids, skip_special_tokens=True))
    if args.show_full_text:
        print("\nprompt and reply together:")
        print(tokenizer.decode(prompt_ids + new_ids, skip_special_tokens=True))
    return 0


if __name__ == "__main__":
    sys.exit(main())
