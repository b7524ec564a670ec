"""Command-line options, declared once per program as a table and parsed in one pass.

The rules are the reference's (apps/options.h:12-62): a name matches exactly or not at all, an
option is a switch or takes exactly one value, naming an option twice or naming one the program
does not have is an error, and a number must lie in its declared range.  Here a program states
name, kind, default and range in one place (`Option`), and `parse` returns every value already
converted and checked, so no call site converts or range-checks again.
"""
from __future__ import annotations

import math
import re
from dataclasses import dataclass
from typing import Optional, Sequence

_INTEGER = re.compile(r"-?[0-9]+")


class OptionError(ValueError):
    pass


@dataclass(frozen=True)
class Option:
    name: str                       # as typed, e.g. "--tokens"
    kind: str = "text"              # "switch", "text", "int", "float" or "ints" (comma-separated integers)
    default: object = None
    low: Optional[float] = None     # inclusive range of an "int" or "float"
    high: Optional[float] = None

    def convert(self, text):
        if self.kind == "text":
            return text
        if self.kind == "int":
            if _INTEGER.fullmatch(text):
                value = int(text)
                if (self.low is None or value >= self.low) and (self.high is None or value <= self.high):
                    return value
            raise OptionError(f"{self.name} {text!r}: not an integer in {self._range()}")
        if self.kind == "float":
            try:
                value = float(text)
            except ValueError:
                value = math.nan
            if math.isfinite(value) and (self.low is None or value >= self.low) and \
                    (self.high is None or value <= self.high):
                return value
            raise OptionError(f"{self.name} {text!r}: not a number in {self._range()}")
        if self.kind == "ints":
            pieces = text.split(",") if text else []
            if all(_INTEGER.fullmatch(piece) for piece in pieces):
                return [int(piece) for piece in pieces]
            raise OptionError(f"{self.name} {text!r}: not a comma-separated list of integers")
        raise OptionError(f"{self.name}: option kind {self.kind!r} is not known")

    def _range(self):
        low = "-inf" if self.low is None else f"{self.low:g}"
        high = "inf" if self.high is None else f"{self.high:g}"
        return f"{low}..{high}"


class Parsed:
    """The values of a command line: `parsed["--tokens"]` (the default where the option was not typed),
    `parsed.given("--tokens")` (whether it was typed)."""

    def __init__(self, values, typed):
        self._values, self._typed = values, typed

    def __getitem__(self, name):
        return self._values[name]

    def given(self, name):
        return name in self._typed


def parse(argv: Sequence[str], table: Sequence[Option]) -> Parsed:
    by_name = {option.name: option for option in table}
    values = {option.name: (False if option.kind == "switch" else option.default) for option in table}
    typed = set()
    words = iter(argv)
    for word in words:
        option = by_name.get(word)
        if option is None:
            raise OptionError(f"{word}: not an option of this program")
        if word in typed:
            raise OptionError(f"{word}: given twice")
        typed.add(word)
        if option.kind == "switch":
            values[word] = True
            continue
        text = next(words, None)
        if text is None:
            raise OptionError(f"{word}: a value must follow")
        values[word] = option.convert(text)
    return Parsed(values, typed)
