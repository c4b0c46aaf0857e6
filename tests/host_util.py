"""Helpers for tests that drive the host runtime without a GPU (dry worlds) and evaluate its traces."""
import re

import numpy as np

from oracle import templates as T

LINE = re.compile(r"rank (\d+) out\[(\d+),(\d+)\) = (.*)")


def parse_trace(text):
    """-> list of (rank, byte offset, byte length, expression string)."""
    out = []
    for line in text.strip().splitlines():
        m = LINE.match(line)
        assert m, line
        out.append((int(m.group(1)), int(m.group(2)), int(m.group(3)), m.group(4)))
    return out


def parse_expr(s):
    """'(a+b)' -> ('+', src, dst); 'xK@B' -> ('x', K, B)."""
    pos = 0

    def rec():
        nonlocal pos
        if s[pos] == "(":
            pos += 1
            a = rec()
            assert s[pos] == "+"
            pos += 1
            b = rec()
            assert s[pos] == ")"
            pos += 1
            return ("+", a, b)
        m = re.match(r"x(\d+)@(\d+)", s[pos:])
        assert m, s[pos:]
        pos += m.end()
        return ("x", int(m.group(1)), int(m.group(2)))

    tree = rec()
    assert pos == len(s)
    return tree


def eval_expr(tree, inputs, nbytes, dtype, op):
    """Evaluates an expression on numpy inputs with the oracle's pairwise element ops: dst = src (+) dst."""
    esz = T.DTYPE_SIZE[dtype]
    if tree[0] == "x":
        _, k, b = tree
        assert b % esz == 0 and nbytes % esz == 0
        return np.ascontiguousarray(inputs[k][b // esz:(b + nbytes) // esz]).copy()
    _, src, dst = tree
    d = eval_expr(dst, inputs, nbytes, dtype, op)
    s = eval_expr(src, inputs, nbytes, dtype, op)
    T.NumericElems(dtype, op).reduce(d, 0, s, 0, d.size)
    return d


def eval_trace(text, inputs, out_elems, dtype, op, fill):
    """Outputs of every rank as the traced expressions define them."""
    esz = T.DTYPE_SIZE[dtype]
    outs = [np.full(out_elems, fill, dtype=inputs[0].dtype) for _ in inputs]
    for rank, off, nbytes, expr in parse_trace(text):
        outs[rank][off // esz:(off + nbytes) // esz] = eval_expr(parse_expr(expr), inputs, nbytes, dtype, op)
    return outs


def expr_to_oracle_string(tree, elem, esz, piece_off):
    """The oracle's symbolic form of element `elem` (index inside the piece)."""
    if tree[0] == "x":
        return f"x{tree[1]}[{tree[2] // esz + elem}]"
    return "(" + expr_to_oracle_string(tree[1], elem, esz, piece_off) + "+" + \
        expr_to_oracle_string(tree[2], elem, esz, piece_off) + ")"


FAKE_IN = 0x100000000000
FAKE_OUT = 0x200000000000
FAKE_STRIDE = 0x001000000000
FAKE_STREAM = 1


def fake_ptrs(n):
    return [FAKE_IN + r * FAKE_STRIDE for r in range(n)], [FAKE_OUT + r * FAKE_STRIDE for r in range(n)]
