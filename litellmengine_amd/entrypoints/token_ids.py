"""Comma-separated token ids, "1,2,3" <-> [1, 2, 3]
(src/runtime/token_ids.cpp:64-109: surrounding spaces are trimmed; an empty
string, an empty item, a sign, a non-digit or a value above int32 is an error)."""
from __future__ import annotations

from typing import List, Sequence

INT32_MAX = 2**31 - 1


def parse_token_ids(text: str) -> List[int]:
    trimmed = text.strip()
    if not trimmed:
        raise ValueError("Token ids string must not be empty")
    out: List[int] = []
    for item in trimmed.split(","):
        item = item.strip()
        if not item:
            raise ValueError("Empty token id in list")
        if not item.isdigit():
            raise ValueError(f"Invalid token id: {item}")
        value = int(item)
        if value > INT32_MAX:
            raise ValueError(f"Token id too large: {item}")
        out.append(value)
    return out


def format_token_ids(ids: Sequence[int]) -> str:
    return ",".join(str(int(i)) for i in ids)
