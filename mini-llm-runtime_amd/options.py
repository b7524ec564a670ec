"""Command-line options in the reference's manner (apps/options.h:12-62): names match exactly,
an option is either a flag or takes one value, an unknown or repeated option is an error, and
numbers are checked against a range."""
from __future__ import annotations

import math


class OptionError(ValueError):
    pass


class Options:
    def __init__(self, argv, values, flags=("--help",)):
        self._args = {}
        values, flags = set(values), set(flags)
        i = 0
        while i < len(argv):
            name = argv[i]
            if name in self._args:
                raise OptionError(f"duplicate option: {name}")
            if name in flags:
                self._args[name] = "true"
            elif name in values and i + 1 < len(argv):
                i += 1
                self._args[name] = argv[i]
            else:
                raise OptionError(f"unknown option or missing value: {name}")
            i += 1

    def has(self, key):
        return key in self._args

    def get(self, key, fallback=""):
        return self._args.get(key, fallback)

    def integer(self, key, fallback, minimum, maximum):
        if not self.has(key):
            return fallback
        text = self.get(key)
        try:
            if text != text.strip() or text.startswith("+"):
                raise ValueError
            value = int(text, 10)
        except ValueError:
            raise OptionError(f"out-of-range integer: {key}") from None
        if value < minimum or value > maximum:
            raise OptionError(f"out-of-range integer: {key}")
        return value

    def number(self, key, fallback, minimum, maximum):
        if not self.has(key):
            return fallback
        try:
            value = float(self.get(key))
        except ValueError:
            raise OptionError(f"out-of-range number: {key}") from None
        if not math.isfinite(value) or value < minimum or value > maximum:
            raise OptionError(f"out-of-range number: {key}")
        return value

    def integers(self, key):
        """A comma-separated list of integers (token ids)."""
        text = self.get(key)
        try:
            return [int(part, 10) for part in text.split(",")] if text else []
        except ValueError:
            raise OptionError(f"not a list of integers: {key}") from None
