"""Reader for the AST text form (test infrastructure; see package docstring).

Independent of the product's C++ parser: a token list and a recursive
descent into nested Python lists.  Atoms stay strings; quoted names become
`Str` instances so they cannot be confused with keywords.
"""

from __future__ import annotations


class Str(str):
    """A double-quoted name from the text."""


def tokenize(text: str):
    out, i, n = [], 0, len(text)
    while i < n:
        c = text[i]
        if c.isspace():
            i += 1
        elif c in "()":
            out.append(c)
            i += 1
        elif c == '"':
            j = text.index('"', i + 1)
            out.append(Str(text[i + 1:j]))
            i = j + 1
        else:
            j = i
            while j < n and not text[j].isspace() and text[j] not in '()"':
                j += 1
            out.append(text[i:j])
            i = j
    return out


def parse(text: str):
    toks = tokenize(text)
    pos = 0

    def rec():
        nonlocal pos
        t = toks[pos]
        pos += 1
        if t == "(" and not isinstance(t, Str):
            lst = []
            while not (toks[pos] == ")" and not isinstance(toks[pos], Str)):
                lst.append(rec())
            pos += 1
            return lst
        return t

    tree = rec()
    if pos != len(toks):
        raise ValueError("trailing tokens after AST text")
    return tree
