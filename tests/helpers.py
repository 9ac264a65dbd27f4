"""Shared helpers for the fixture-driven tests: the text forms used by tests/golden/*.json."""
import json
import os
import re

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load_vectors():
    with open(os.path.join(GOLDEN, "layout_vectors.json")) as f:
        return json.load(f)


def canon(text):
    """Expand the `@` shorthand: every integer of the argument becomes static (`_n`)."""
    text = text.strip()
    if text.startswith("<"):
        return "<" + ",".join(canon(p) for p in split_top(text[1:-1])) + ">"
    if not text.startswith("@"):
        return text
    return re.sub(r"(?<![_\d])(-?\d+)", r"_\1", text[1:])


def split_top(text):
    """Split on commas that are not inside parentheses or angle brackets."""
    out, depth, cur = [], 0, ""
    for ch in text:
        if ch in "(<":
            depth += 1
        elif ch in ")>":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur)
            cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur)
    return [p.strip() for p in out]
