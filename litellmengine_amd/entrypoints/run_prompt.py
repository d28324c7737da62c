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


def main(argv=None) -> int:
    p = argparse.ArgumentParser(prog="run_prompt")
    p.add_argument("--model", required=True)
    p.add_argument("--engine", default=None, help="engine executable (default: call the engine in-process)")
    p.add_argument("--prompt", required=True)
    p.add_argument("--max-tokens", type=int, default=64)
    p.add_argument("--device", default="cuda")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--eos-token-id", type=int, default=None, help="default: the tokenizer's <|im_end|>")
    p.add_argument("--no-chat-template", action="store_true")
    p.add_argument("--show-full-text", action="store_true")
    args = p.parse_args(argv)

    import os

    from tokenizers import Tokenizer

    tokenizer = Tokenizer.from_file(os.path.join(args.model, "tokenizer.json"))
    input_ids = encode_prompt(tokenizer, args.model, args.prompt, not args.no_chat_template)
    eos = args.eos_token_id
    if eos is None:
        eos = tokenizer.token_to_id("<|im_end|>")
    ids_text = ",".join(map(str, input_ids))
    print("[run_prompt] input ids:")
    print(ids_text)
    print("len =", len(input_ids))
    print()

    if args.engine:
        cmd = [args.engine, "--model", args.model, "--input-ids", ids_text, "--max-tokens", str(args.max_tokens),
               "--device", args.device, "--temperature", "0", "--dtype", args.dtype]
        if eos is not None:
            cmd += ["--eos-token-id", str(eos)]
        result = subprocess.run(cmd, text=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, check=False)
        print("[engine output]")
        print(result.stdout)
        if result.returncode != 0:
            return result.returncode
        new_ids = parse_new_token_ids(result.stdout)
    else:
        from .generate import generate

        new_ids = generate(args.model, [input_ids], args.max_tokens, 0.0, -1 if eos is None else eos,
                           args.dtype, args.device)[0]
    print("[decoded new text]")
    print(tokenizer.decode(new_ids, skip_special_tokens=True))
    if args.show_full_text:
        print()
        print("[decoded full text]")
        print(tokenizer.decode(input_ids + new_ids, skip_special_tokens=True))
    return 0


if __name__ == "__main__":
    sys.exit(main())
