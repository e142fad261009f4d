"""Pretty-printing of a HipTensor in the reference's formats.

`pretty(t)` / `str(t)` is what `echo cudaTensor` is in the reference
(src/arraymancer/tensor/display_cuda.nim:19-36): the tensor is brought to the host and laid out by
the CPU printer (src/arraymancer/tensor/display.nim:19-115, private/p_display.nim:152-485):

  * table mode (the default, specifier "" or "||" / "<|>" / "<>||"): a header line, then the last
    two dimensions as rows between `|`, odd dimensions stacked horizontally with their index
    centred above, even dimensions stacked vertically with their index centred on the left;
  * array modes: "[]" one line, "[:]" one row per line, with "<>" / "<:>" a compact header.

Floats print like C's "%g" (precision -1) or "%#.{precision}g"; integers in decimal; bools as
true / false. The text is produced on the host from the values copied back; nothing here computes
on tensors.
"""
from __future__ import annotations

import numpy as np

# Nim's names of the element types (int and float are the 64-bit ones on this platform).
_TYPE_NAME = {np.dtype(np.float32): "float32", np.dtype(np.float64): "float", np.dtype(np.int32): "int32",
              np.dtype(np.int64): "int", np.dtype(np.bool_): "bool", np.dtype(np.uint8): "uint8"}


def _elem(v, precision: int) -> str:
    if isinstance(v, (bool, np.bool_)):
        return "true" if v else "false"
    if isinstance(v, (float, np.floating)):
        v = float(v)
        if v != v:
            return "nan"
        if v in (float("inf"), float("-inf")):
            return "inf" if v > 0 else "-inf"
        return ("%#.*g" % (precision, v)) if precision >= 0 else ("%g" % v)
    return str(int(v))


def _center(s: str, width: int) -> str:
    """Nim's strutils.center: the left padding is the smaller one."""
    if width <= len(s):
        return s
    left = (width - len(s)) // 2
    return " " * left + s + " " * (width - len(s) - left)


def _zip_strings(s1: str, s2: str, sep: str = "", allow_empty: bool = False) -> str:
    a, b = s1.split("\n"), s2.split("\n")
    if len(a) == 1:
        return s2
    if len(b) == 1:
        return s1
    out = []
    for x, y in zip(a, b):
        if not allow_empty and not x and not y:
            continue
        out.append(x + sep + y + "\n")
    return "".join(out)


def _gen_sep(rank: int, line_len: int = 0, xaxis: bool = False) -> str:
    out = ""
    for i in range(2, rank):
        if i % 2 == 0:
            out += "-" * line_len if xaxis else " "
        else:
            out += " " * line_len if xaxis else " | "
        if xaxis:
            out += "\n"
    return out


def _left_idx(ax_idx: str, s: str) -> str:
    tmp = _center(ax_idx + " ", len(s.split("\n"))).split(" ")
    out = ""
    high = len(tmp) - 1
    for i in range(high):
        out += (tmp[i] + " ") if tmp[i] else (" " * len(ax_idx) + " ")
        if i < high - 1:
            out += "\n"
    return out


def _disp2d(a: np.ndarray, align_by: int, align_spacing: int, precision: int) -> str:
    """Rows of a matrix between `|` (a vector: one run of right-aligned cells)."""
    cols = a.shape[-1] if a.ndim == 2 else None
    out = []
    for idx, v in enumerate(a.reshape(-1), start=1):
        val = _elem(v, precision)
        if cols is None:
            out.append(val.rjust(align_by))
        elif idx % cols == 0:
            if cols == 1:
                out.append("|" + val.rjust(align_by - align_spacing) + "|\n")
            else:
                out.append(val.rjust(align_by) + "|\n")
        elif idx % cols == 1:
            out.append("|" + val.ljust(align_by - align_spacing))
        else:
            out.append(val.rjust(align_by))
    return "".join(out)


def _squeeze(a: np.ndarray) -> np.ndarray:
    s = a.squeeze()
    return s.reshape(1) if s.ndim == 0 else s


def _table(a: np.ndarray, input_rank: int = 0, align_by: int = 0, precision: int = -1) -> str:
    align_spacing = 4
    if input_rank == 0:
        input_rank = a.ndim
        largest = max((len(_elem(v, precision)) for v in a.reshape(-1)), default=0)
        align_by = max(6, largest + align_spacing)
    if a.ndim <= 2:
        return _disp2d(a, align_by, align_spacing, precision).strip()
    res = ""
    odd = a.ndim % 2 != 0
    for ax_idx in range(a.shape[0]):
        sub = _table(_squeeze(a[ax_idx:ax_idx + 1]), input_rank, align_by, precision)
        if odd:     # next "column": its index centred above it, zipped to the right of what is there
            sub = _center(str(ax_idx), len(sub.split("\n")[0])) + "\n" + sub
            res = _zip_strings(res, sub, sep=_gen_sep(a.ndim), allow_empty=False)
        else:       # next "row": its index centred on the left, stacked below
            res += _zip_strings(_left_idx(str(ax_idx), sub), sub, allow_empty=True)
    if odd and a.ndim != input_rank:
        res += _gen_sep(a.ndim, len(res.split("\n")[0]), True)
    return res


def _array_line(a: np.ndarray, precision: int, row_sep: str) -> str:
    if a.ndim <= 1:
        return "[" + ", ".join(_elem(v, precision) for v in a.reshape(-1)) + "]"
    parts = []
    for i in range(a.shape[0]):
        sub = a[i:i + 1]
        if sub.shape[0] == 1:                     # squeezeTopDimension
            sub = sub.reshape(sub.shape[1:])
        parts.append(_array_line(sub, precision, row_sep))
    return "[" + (", " + row_sep).join(parts) + "]"


def _indent_rows(s: str, rank: int) -> str:
    out = []
    for line in s.split("\n"):
        brackets = len(line) - len(line.lstrip("["))
        out.append(" " * max(rank - brackets, 0) + line if line else line)
    return "\n".join(out).rstrip()


def _parse(specifier: str):
    """(mode, header) of the tensor-specific part of a format specifier; element format
    specifiers beyond `precision` are not supported."""
    table = {"": ("table", True), "||": ("table", False), "<|>": ("table", True), "<>||": ("table", True),
             "[]": ("single", False), "<>[]": ("single", True), "<>": ("single", True),
             "[:]": ("multi", False), "<>[:]": ("multi", True), "<:>": ("multi", True)}
    if specifier not in table:
        raise ValueError(f"Invalid tensor format specifier ({specifier}): one of {sorted(table)} expected")
    return table[specifier]


def pretty_array(host: np.ndarray, type_name: str, backend: str, precision: int = -1, specifier: str = "") -> str:
    """The reference's prettyImpl (private/p_display.nim:452-485) for a host array."""
    mode, header = _parse(specifier)
    shape = list(host.shape)
    elem = _TYPE_NAME.get(host.dtype, str(host.dtype))
    if mode != "table":
        compact = f"{type_name}[{elem}]<{','.join(str(s) for s in shape)}>"
        if mode == "single":
            return (compact + ":" if header else "") + _array_line(host, precision, "")
        body = _indent_rows(_array_line(host, precision, "\n"), host.ndim)
        return (compact + ":\n" if header else "") + body
    desc = f'{type_name}[system.{elem}] of shape "{shape}" on backend "{backend}"\n' if header else ""
    if host.size == 0:
        return desc + "    [] (empty)"
    if host.ndim == 1:
        return desc + "    " + _table(host, precision=precision)
    return desc + _table(host, precision=precision)
