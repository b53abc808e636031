"""Shared pieces of the gfx950 kernel generator: source emitter, literals, Jinja environment."""
from __future__ import annotations

import pathlib
from typing import Iterable, List

import jinja2
import numpy as np

TEMPLATE_DIR = pathlib.Path(__file__).resolve().parent / "templates"
WAVE = 64


def jinja_env() -> jinja2.Environment:
    env = jinja2.Environment(loader=jinja2.FileSystemLoader(str(TEMPLATE_DIR)),
                             trim_blocks=True, lstrip_blocks=True, undefined=jinja2.StrictUndefined,
                             keep_trailing_newline=True)
    env.globals.update(enumerate=enumerate, len=len, range=range, zip=zip)
    return env


def literal(value: float, ctype: str) -> str:
    """Exact hexadecimal floating literal of ``value`` rounded to the kernel's precision."""
    if ctype == "float":
        return float(np.float32(value)).hex() + "f"
    return float(value).hex()


def next_pow2(n: int) -> int:
    p = 1
    while p < n:
        p *= 2
    return p


class Emitter:
    """Accumulates indented source lines."""

    def __init__(self, indent: int = 1):
        self.lines: List[str] = []
        self.level = indent

    def __call__(self, text: str = "") -> None:
        for line in text.split("\n"):
            self.lines.append(("    " * self.level + line) if line else "")

    def open(self, head: str) -> None:
        self(head + " {")
        self.level += 1

    def close(self, tail: str = "") -> None:
        self.level -= 1
        self("}" + tail)

    def extend(self, lines: Iterable[str]) -> None:
        for l in lines:
            self(l)

    def text(self) -> str:
        return "\n".join(self.lines)
