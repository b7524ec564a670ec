"""Text in and out.  The engine works on token ids; this is the thin wrapper that the command line's
--prompt and the Python entry point's text prompts go through, as the reference wraps its vocabulary
library (src/minillm/tokenizer.cpp:14-72: a vocabulary checked against the embedding matrix, `tokenize`,
`token_piece`, `is_eog`).  The vocabulary is a model folder's `tokenizer.json`, read by the `tokenizers`
package; nothing here is needed, or imported, while prompts are given as ids."""
from __future__ import annotations

import os

MAX_PROMPT_BYTES = 262144        # src/minillm/tokenizer.cpp:42-44


class TokenizerError(ValueError):
    pass


def tokenizer_file(path):
    """`path` itself when it is a file, else the tokenizer.json inside that folder (or None)."""
    if os.path.isfile(path):
        return path
    inside = os.path.join(path, "tokenizer.json")
    return inside if os.path.isfile(inside) else None


class Tokenizer:
    def __init__(self, path, expected_vocabulary, eog_ids=()):
        """`path`: a tokenizer.json or the folder that holds one.  `expected_vocabulary`: the rows of the
        embedding matrix; every id the vocabulary knows must be one of them (a model's matrix may have more
        rows than its vocabulary has entries: they are padding).  `eog_ids`: the ids that end a generation."""
        file = tokenizer_file(path)
        if file is None:
            raise TokenizerError(f"no tokenizer.json in {path}: give prompts as token ids, or name one with --tokenizer")
        try:
            import tokenizers
        except ImportError:
            raise TokenizerError("text prompts need the `tokenizers` package; give prompts as token ids") from None
        try:
            self._tok = tokenizers.Tokenizer.from_file(file)
        except Exception as error:
            raise TokenizerError(f"cannot load the tokenizer {file}: {error}") from None
        self.path = file
        known = self._tok.get_vocab(with_added_tokens=True)
        self._size = len(known)
        highest = max(known.values(), default=-1)
        if highest >= expected_vocabulary:
            raise TokenizerError(f"tokenizer vocabulary does not fit the embedding matrix: it names id {highest}, "
                                 f"the matrix has {expected_vocabulary} rows")
        self._eog = frozenset(int(t) for t in eog_ids)

    def vocabulary_size(self):
        return self._size

    def tokenize(self, text):
        """Ids of `text`, with the vocabulary's own leading and trailing special tokens where it adds any and
        special tokens written out in the text taken as such (src/minillm/tokenizer.cpp:46-47)."""
        if len(text.encode("utf-8")) > MAX_PROMPT_BYTES:
            raise TokenizerError("prompt exceeds 256 KiB")
        return list(self._tok.encode(text, add_special_tokens=True).ids)

    def token_piece(self, token):
        """The text of one token; nothing for a special token (src/minillm/tokenizer.cpp:58-59)."""
        return self._tok.decode([int(token)], skip_special_tokens=True)

    def text(self, tokens):
        """The text of a run of tokens, special tokens left out.  (Decoded as a whole: a character that a
        byte-level vocabulary spreads over several tokens comes out whole.)"""
        return self._tok.decode([int(t) for t in tokens], skip_special_tokens=True)

    def is_eog(self, token):
        return int(token) in self._eog
