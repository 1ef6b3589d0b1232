"""Connector-name helpers (API of ``daceml/onnx/nodes/node_utils.py``).

A variadic ONNX parameter ``name`` shows up on a node as connectors ``name__0``,
``name__1``, ...: the index is a canonical non-negative decimal.
"""
import re
import typing

_VARIADIC = re.compile(r"(?P<base>[^_](?:.*[^_])?)__(?P<index>[^_].*|)")
_CANONICAL_INDEX = re.compile(r"0|[1-9][0-9]*")


def is_variadic_connector(connector: str) -> bool:
    return "__" in connector


def parse_variadic_param(param: str) -> typing.Tuple[str, int]:
    """``"name__3"`` -> ``("name", 3)``; ValueError for anything that is not of that form."""
    match = _VARIADIC.fullmatch(param)
    if match is None or "__" in match["base"] or "__" in match["index"]:
        raise ValueError(f"Unable to parse variadic parameter '{param}'")
    index = match["index"]
    if not _CANONICAL_INDEX.fullmatch(index):
        if index.isdigit():
            raise ValueError(f"Variadic parameters must not be numbered with leading zeroes, got: '{index}'")
        raise ValueError(f"Variadic parameters must be numbered with non-negative integers, got: '{index}'")
    return match["base"], int(index)
